"""Mixers side by side: every branch reads the same input, the result is the sum of the branches'
results, each times a constant of its own.

A branch is any registered mixer that takes `out_scale` (it applies the constant itself, in float32,
before its output product) and adds into the `residual` it is given: the first branch's output product
writes the sum's buffer, every further one adds to it, so the sum costs no kernel of its own.  At most one
branch may keep a paged cache and at most one a per-request state; they become the part's own.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from .base import MIXERS, CacheSpec, Mixer, StateSpec, WeightSpec, register_mixer


class ParallelMixer(Mixer):
    def __init__(self, prefix, dtype, device, *, branches: Sequence[dict]):
        """branches: [{"kind": registered mixer, "name": weight-name component, "scale": constant,
        "params": the mixer's own parameters}, ...]"""
        super().__init__(prefix, dtype, device)
        if not branches:
            raise ValueError(f"{prefix}: a parallel mixer needs at least one branch")
        self.branches: List[Mixer] = []
        for b in branches:
            params = dict(b.get("params") or {})
            params["out_scale"] = float(b.get("scale", 1.0))
            self.branches.append(MIXERS.get(b["kind"])(f"{prefix}.{b['name']}", dtype, device, **params))
        with_cache = [m for m in self.branches if m.cache_spec() is not None]
        with_state = [m for m in self.branches if m.state_spec() is not None]
        if len(with_cache) > 1 or len(with_state) > 1:
            raise ValueError(f"{prefix}: at most one branch may keep a cache and at most one a state")
        self._cache_branch = with_cache[0] if with_cache else None
        self._state_branch = with_state[0] if with_state else None

    @property
    def graph_safe(self) -> bool:
        parts = list(self.branches) + [getattr(m, "position", None) for m in self.branches]
        return all(p.graph_safe for p in parts if p is not None)

    def weights(self) -> List[WeightSpec]:
        return [w for m in self.branches for w in m.weights()]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        for m in self.branches:
            m.bind(tensors)

    def cache_spec(self) -> Optional[CacheSpec]:
        return self._cache_branch.cache_spec() if self._cache_branch is not None else None

    def state_spec(self) -> Optional[StateSpec]:
        return self._state_branch.state_spec() if self._state_branch is not None else None

    def forward(self, h, ctx, cache, state, residual):
        y = residual
        for m in self.branches:
            y = m.forward(h, ctx, cache if m is self._cache_branch else None,
                          state if m is self._state_branch else None, y)
        return y


register_mixer("parallel", ParallelMixer)
