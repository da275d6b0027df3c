"""Rotary position encoding: the angle tables and the pairing.

theta[p, i] = p * base^(-i / (rotary_dim/2)), computed in float64 and rounded to
float32 cos / sin tables of shape [max_position, rotary_dim/2], as the reference
does (tiny_llm/ops/cuda/rope.cu:12-24).  The rotation itself (the reference's
rotate-half pairing (i, i + rotary_dim/2), rope.cu:46-54) is fused with the cache
write in the attention mixer's kernels; this part owns the constants:
(theta, rotary_dim, pairing, scaling).

pairing  "half" (the reference's) or "interleaved" (pair i is the dims 2i, 2i + 1).
scaling  None, or {"kind": "linear", "factor": f}: positions are divided by f before the
         angles are taken (the table changes, nothing else); or {"kind": "yarn", "factor": s,
         "original": L, "fast": b, "slow": a}: frequency by frequency a blend between f_i and
         f_i / s, and cos and sin times 0.1 ln(s) + 1 (see `yarn_frequencies`).  Other kinds are
         refused by name.
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Tuple

import torch

from .base import PositionEncoding, register_position_encoding

# Angle tables by (rotary_dim, theta, max_position, position factor, device): the layers of a model share one pair.
_TABLES: Dict[Tuple, Tuple[torch.Tensor, torch.Tensor]] = {}

PAIRINGS = ("half", "interleaved")
SCALINGS = ("linear", "yarn")


def yarn_frequencies(inv_freq: torch.Tensor, rotary_dim: int, theta: float, factor: float, original: float,
                     fast: float, slow: float) -> Tuple[torch.Tensor, float]:
    """YaRN: frequencies that turn more than `fast` times within `original` positions stay, those
    that turn fewer than `slow` times are divided by `factor`, the ones between are blended.
    With n(t) = rotary_dim * ln(original / (2 pi t)) / (2 ln theta) (the index whose frequency turns t
    times), lo = max(floor(n(fast)), 0), hi = min(ceil(n(slow)), rotary_dim - 1) and
    r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1):  f_i' = r_i f_i / factor + (1 - r_i) f_i.
    Returns (f', the factor 0.1 ln(factor) + 1 for cos and sin)."""
    def index_of(turns: float) -> float:
        return rotary_dim * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(theta))

    lo = max(math.floor(index_of(fast)), 0)
    hi = min(math.ceil(index_of(slow)), rotary_dim - 1)
    i = torch.arange(inv_freq.numel(), dtype=torch.float64)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return inv_freq / factor * ramp + inv_freq * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def angle_tables(rotary_dim: int, theta: float, max_position: int, device, position_factor: float = 1.0,
                 yarn: Optional[Tuple[float, float, float, float]] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """float32 (cos, sin) [max_position, rotary_dim / 2] of theta[p, i] = (p / position_factor) *
    base^(-i / (rotary_dim / 2)), computed in float64 on the host (tiny_llm/ops/cuda/rope.cu:12-24,
    which has no factor).  yarn = (factor, original, fast, slow): frequencies and magnitude of
    `yarn_frequencies`."""
    key = (int(rotary_dim), float(theta), int(max_position), float(position_factor), yarn,
           str(torch.device(device)))
    if key not in _TABLES:
        half = rotary_dim // 2
        idx = torch.arange(half, dtype=torch.float64)
        inv_freq = torch.pow(torch.tensor(float(theta), dtype=torch.float64), -idx / half)
        magnitude = 1.0
        if yarn is not None:
            inv_freq, magnitude = yarn_frequencies(inv_freq, rotary_dim, theta, *yarn)
        pos = torch.arange(max_position, dtype=torch.float64)
        if position_factor != 1.0:
            pos = pos / float(position_factor)
        ang = pos[:, None] * inv_freq[None, :]
        _TABLES[key] = ((torch.cos(ang) * magnitude).to(torch.float32).contiguous().to(device),
                        (torch.sin(ang) * magnitude).to(torch.float32).contiguous().to(device))
    return _TABLES[key]


class RotaryEmbedding(PositionEncoding):
    graph_safe = True

    def __init__(self, prefix, dtype, device, *, head_dim: int, theta: float, max_position: int,
                 rotary_dim: int = None, pairing: str = "half", scaling: dict = None):
        super().__init__(prefix, dtype, device)
        if pairing not in PAIRINGS:
            raise ValueError(f"rotary pairing {pairing!r} is not built; known: {', '.join(PAIRINGS)}")
        self.pairing = pairing
        factor, yarn = 1.0, None
        if scaling is not None:
            kind = dict(scaling).get("kind")
            if kind not in SCALINGS:
                raise ValueError(f"rotary scaling {kind!r} is not built; known: {', '.join(SCALINGS)}")
            if not float(scaling["factor"]) > 0:
                raise ValueError("the factor of rotary scaling must be positive")
            if kind == "linear":
                factor = float(scaling["factor"])
            else:
                yarn = tuple(float(scaling[k]) for k in ("factor", "original", "fast", "slow"))
                if not (yarn[1] > 0 and yarn[2] > 0 and yarn[3] > 0):
                    raise ValueError("yarn scaling needs positive `original`, `fast` and `slow`")
        self.position_factor = factor
        self.yarn = yarn
        self.head_dim = int(head_dim)
        self.rotary_dim = int(head_dim if rotary_dim is None else rotary_dim)
        if self.rotary_dim % 2 or not (0 < self.rotary_dim <= self.head_dim):
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within head_dim {self.head_dim}")
        self.theta = float(theta)
        self.max_position = int(max_position)
        self.cos, self.sin = angle_tables(self.rotary_dim, self.theta, self.max_position, device, factor, yarn)

    def rotary_tables(self):
        return self.cos, self.sin, self.rotary_dim


class NoPositionEncoding(PositionEncoding):
    graph_safe = True

    def __init__(self, prefix, dtype, device, **_):
        super().__init__(prefix, dtype, device)


register_position_encoding("rotary", RotaryEmbedding)
register_position_encoding("none", NoPositionEncoding)
