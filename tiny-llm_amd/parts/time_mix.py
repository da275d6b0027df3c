"""Time mixing with a decaying matrix state per head: a recurrent mixer.

Per token, with h the mixer's input and h' the previous token's (zeros before a request's first):
    m_s  = h + (h' - h) * mu_s                       one mix per projection, s in r, k, v, g, w
    r, k, v = W_r m_r, W_k m_k, W_v m_v              heads x dim each
    gate = silu(W_g m_g)
    w    = exp(-exp(W_w2 tanh(W_w1 m_w) + w0))       a decay per head and key channel
    per head:  o = (S + diag(u) k v^T)^T r,  then  S <- diag(w) S + k v^T      (u: a bonus for the current token)
    out  = out_scale * W_o (unit_rms(o) per head * w_norm * gate)
Per request the part keeps S of every head and the last token's h in ONE float32 state row, which the
cache manager zeroes when the request is admitted.  The products' results stay float32 on their way into
the recurrence; decays, the state, the head norm and the gate are float32 in both precisions.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from ..kernels import ops
from .base import Mixer, StateSpec, WeightSpec, register_mixer


def _pad8(n: int) -> int:
    return -(-n // 8) * 8


class TimeMix(Mixer):
    graph_safe = True
    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, prefix, dtype, device, *, hidden_size: int, num_heads: int, head_dim: int, decay_rank: int,
                 eps: float, out_scale: float = 1.0, names: Dict[str, str] = None):
        super().__init__(prefix, dtype, device)
        self.hidden_size, self.num_heads, self.head_dim = int(hidden_size), int(num_heads), int(head_dim)
        self.decay_rank, self.eps, self.out_scale = int(decay_rank), float(eps), float(out_scale)
        if self.num_heads <= 0 or not (0 < self.head_dim <= ops.TIME_MIX_MAX_DIM):
            raise ValueError(f"{prefix}: heads of 1 to {ops.TIME_MIX_MAX_DIM} channels, got {self.num_heads} x {self.head_dim}")
        if self.decay_rank <= 0:
            raise ValueError(f"{prefix}: the rank of the decay's projection must be positive")
        self.size = self.num_heads * self.head_dim
        ops.check_linear_sizes(dtype, self.hidden_size, f"{prefix}: hidden_size")
        ops.check_linear_sizes(dtype, self.size, f"{prefix}: heads * dim")
        self.seg = _pad8(self.size)                      # r | k | v | decay, each from a multiple of 8 columns
        self.rank = _pad8(self.decay_rank)
        self.s_floats = ops.time_mix_state_floats(self.num_heads, self.head_dim, self.head_dim)
        n = {k: k for k in ("r", "k", "v", "g", "w1", "w2", "w0", "u", "norm", "o")}
        n.update({f"mu.{k}": f"mu.{k}" for k in self.MIXES})
        n.update(names or {})
        self.names = {k: f"{prefix}.{v}" for k, v in n.items()}
        self.mu = self.w_r = self.w_k = self.w_v = self.w_g = self.w1 = self.w2 = self.w_o = None
        self.w0 = self.u = self.w_norm = None

    def weights(self) -> List[WeightSpec]:
        n, W, S = self.names, self.hidden_size, self.size
        vec = dict(role="vector")
        out = [WeightSpec(n[f"mu.{k}"], (W,), **vec) for k in self.MIXES]
        out += [WeightSpec(n[k], (S, W)) for k in ("r", "k", "v", "g")]
        out += [WeightSpec(n["w1"], (self.decay_rank, W)), WeightSpec(n["w2"], (S, self.decay_rank)),
                WeightSpec(n["w0"], (S,), **vec), WeightSpec(n["u"], (self.num_heads, self.head_dim), **vec),
                WeightSpec(n["norm"], (S,), role="vector", init="ones"), WeightSpec(n["o"], (W, S))]
        return out

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        n = self.names
        f32 = lambda t: t.to(torch.float32).contiguous()
        self.mu = torch.stack([f32(tensors[n[f"mu.{k}"]]) for k in self.MIXES]).contiguous()
        self.w_r, self.w_k, self.w_v, self.w_g = (tensors[n[k]].contiguous() for k in ("r", "k", "v", "g"))
        dev = self.w_r.device
        w1 = torch.zeros((self.rank, self.hidden_size), dtype=self.dtype, device=dev)
        w1[:self.decay_rank] = tensors[n["w1"]]
        w2 = torch.zeros((self.size, self.rank), dtype=self.dtype, device=dev)
        w2[:, :self.decay_rank] = tensors[n["w2"]]
        self.w1, self.w2 = w1, w2
        self.w0, self.w_norm = f32(tensors[n["w0"]]), f32(tensors[n["norm"]])
        self.u = f32(tensors[n["u"]]).reshape(-1)
        self.w_o = tensors[n["o"]].contiguous()

    def state_spec(self) -> StateSpec:
        # [S in the recurrence kernel's layout | the last token's h], rows a multiple of four floats
        return StateSpec((-(-(self.s_floats + self.hidden_size) // 4) * 4,), torch.float32)

    def forward(self, h, ctx, cache, state, residual):
        T, dev, S, seg = h.shape[0], h.device, self.size, self.seg
        mixes = ops.scratch("shift_mixes", (len(self.MIXES), T, self.hidden_size), self.dtype, dev)
        single = ctx.max_q_len == 1              # no request brings more than one token: the shift saves it itself
        ops.shift_mix(h, state, self.s_floats, ctx.req_of_token, ctx.cu_seqlens_q, ctx.state_slots, self.mu, mixes,
                      save_single=single)
        if not single:
            ops.shift_save(h, state, self.s_floats, ctx.cu_seqlens_q, ctx.state_slots)
        x = ops.scratch("time_mix_in", (T, 4 * seg), torch.float32, dev)
        ops.linear(mixes[0], self.w_r, x[:, 0:S])
        ops.linear(mixes[1], self.w_k, x[:, seg:seg + S])
        ops.linear(mixes[2], self.w_v, x[:, 2 * seg:2 * seg + S])
        gate = ops.scratch("time_mix_gate", (T, S), torch.float32, dev)
        ops.linear(mixes[3], self.w_g, gate)
        low = ops.scratch("time_mix_low", (T, self.rank), torch.float32, dev)
        ops.linear(mixes[4], self.w1, low)
        act = ops.tanh_rows(low, ops.scratch("time_mix_low_act", (T, self.rank), self.dtype, dev))
        ops.linear(act, self.w2, x[:, 3 * seg:3 * seg + S])
        o = ops.scratch("time_mix_o", (T * S,), torch.float32, dev)
        ops.time_mix_recurrence(x, 0, seg, 2 * seg, 3 * seg, self.w0, self.u, state, ctx.cu_seqlens_q, ctx.state_slots, o,
                                self.num_heads, self.head_dim, self.head_dim)
        z = ops.scratch("time_mix_gated", (T, S), self.dtype, dev)
        ops.head_norm_gate(o, self.w_norm, gate, z, self.num_heads, self.head_dim, self.eps, "silu", self.out_scale)
        if residual is None:
            return ops.linear(z, self.w_o, ops.scratch("sublayer_out", (T, self.hidden_size), torch.float32, dev))
        return ops.linear(z, self.w_o, residual, residual)


register_mixer("time_mix", TimeMix)
