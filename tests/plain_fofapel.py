"""A plain, slow Fofapel: every mechanism of the design as one small function, written from its
equations with torch on the CPU (float64 unless told otherwise).  It shares no code with the
engine: it reads config.json's own keys and the checkpoint's tensor names, keeps whole sequences
(no cache, no pages, no state slots) and runs one request at a time.

Notation: x [T, W] is the residual stream; a sublayer reads x itself and the layer's norm follows
the sum (x <- LN(alpha x + f(x))); weights are [out, in] and applied as h @ W.T.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


# --------------------------------------------------------------------------- norms
def layer_norm(x, w, b, eps):
    """(x - mean) / sqrt(var + eps) * w + b, var the mean squared deviation, over the last axis."""
    mu = x.mean(dim=-1, keepdim=True)
    d = x - mu
    return d / torch.sqrt((d * d).mean(dim=-1, keepdim=True) + eps) * w + b


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis, no weight."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# ------------------------------------------------------------------------ rotation
def rotate_pairs(x, positions, dims: int, base: float):
    """x [T, heads, D]: of the last axis the first `dims` rotate, element 2i paired with 2i + 1,
    by the angle p * base^(-2i/dims); the rest passes."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    a = positions.to(torch.float64)[:, None] * f[None, :]
    cos, sin = torch.cos(a)[:, None, :].to(x.dtype), torch.sin(a)[:, None, :].to(x.dtype)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


# ---------------------------------------------------- windowed attention with a sink
def sink_softmax(s, allowed):
    """p_j = exp(s_j) / (1 + sum_allowed exp(s_j)): a sink of score 0 that carries no value."""
    s = s.masked_fill(~allowed, float("-inf"))
    m = torch.clamp(s.max(dim=-1, keepdim=True).values, min=0.0)
    e = torch.exp(s - m)
    return e / (torch.exp(-m) + e.sum(dim=-1, keepdim=True))


def window_attention(h, w, m, eps, positions):
    """The left mixer.  h [T, W] -> [T, W].  Values are the keys as projected."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ w["q"].T + w["q.b"]).reshape(T, H, D)
    k = (h @ w["k"].T + w["k.b"]).reshape(T, G, D)
    v = k
    rot = m.get("rot")
    if rot:
        q = rotate_pairs(q, positions, rot["dims"], rot["base"])
        k = rotate_pairs(k, positions, rot["dims"], rot["base"])
    q, k = rms_unit(q, eps), rms_unit(k, eps)
    i, j = positions[:, None], positions[None, :]
    allowed = (j <= i) & (i - j < m["mask"]["size"])
    gate = torch.sigmoid(h @ w["g"].T)                         # [T, H]
    out = torch.zeros(T, H, D, dtype=h.dtype)
    for n in range(H):
        g = n // (H // G)
        s = (q[:, n] @ k[:, g].T) * m["scale"]
        out[:, n] = sink_softmax(s, allowed) @ v[:, g]
    out = out * gate[:, :, None]
    return out.reshape(T, H * D) @ w["o"].T


# ------------------------------------------------------- time mixing with a decaying state
def shifted_mix(h, mu):
    """h + (h_prev - h) * mu, h_prev the row before (zeros before the first)."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)
    return h + (prev - h) * mu


def decay_of(mix_w, w1, w2, w0):
    """exp(-exp(W2 tanh(W1 mix) + w0)): one factor in (0, 1) per head and key channel."""
    return torch.exp(-torch.exp(torch.tanh(mix_w @ w1.T) @ w2.T + w0))


def time_mix_recurrence(r, k, v, decay, u):
    """Per head, state S [D, D] from zero:  o_t = (S + diag(u) k_t v_t^T)^T r_t, then
    S <- diag(decay_t) S + k_t v_t^T.   r, k, v, decay [T, H, D]; u [H, D] -> o [T, H, D]."""
    T, H, D = r.shape
    S = torch.zeros(H, D, D, dtype=r.dtype)
    o = torch.zeros(T, H, D, dtype=r.dtype)
    for t in range(T):
        kv = k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hd,hde->he", r[t], S + u[:, :, None] * kv)
        S = decay[t][:, :, None] * S + kv
    return o


def time_mix(h, w, m, eps):
    """The right mixer.  h [T, W] -> [T, W]."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    r = (shifted_mix(h, w["mu.r"]) @ w["r"].T).reshape(T, H, D)
    k = (shifted_mix(h, w["mu.k"]) @ w["k"].T).reshape(T, H, D)
    v = (shifted_mix(h, w["mu.v"]) @ w["v"].T).reshape(T, H, D)
    gz = shifted_mix(h, w["mu.g"]) @ w["g"].T
    gate = gz * torch.sigmoid(gz)
    decay = decay_of(shifted_mix(h, w["mu.w"]), w["w1"], w["w2"], w["w0"]).reshape(T, H, D)
    o = time_mix_recurrence(r, k, v, decay, w["u"])
    o = rms_unit(o, eps).reshape(T, H * D) * w["norm"] * gate
    return o @ w["o"].T


def parallel_mixer(h, w, m, eps, positions):
    left = window_attention(h, _sub(w, "left."), m["left"], eps, positions)
    right = time_mix(h, _sub(w, "right."), m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


# -------------------------------------------------------------------- feed-forwards
def dense_ff(h, w):
    return (gelu_tanh(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def clamped_expert(h, w, limit):
    g = torch.clamp(h @ w["gate"].T, max=limit)
    u = torch.clamp(h @ w["up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w["down"].T


def table_moe(h, w, mlp, tokens):
    """Every token's experts come from a table row of its id; each weighs 1 / top.  A shared
    expert, if the layer has one, is added, times sigmoid(w_sg . h) if it has a gate."""
    top = mlp["router"]["top"]
    table = w["table"].to(torch.long)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in table[int(tokens[t])].tolist():
            out[t] += clamped_expert(h[t:t + 1], _sub(w, f"e{e}."), mlp["expert"]["limit"])[0] / top
    if mlp.get("shared"):
        s = _sub(w, "shared.")
        y = clamped_expert(h, s, mlp["shared"]["limit"])
        out = out + (y * torch.sigmoid(h @ s["sg"].T) if "sg" in s else y)
    return out


# ---------------------------------------------------------------------------- model
def _sub(w: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}


def layer_forward(cfg, w, i: int, x, tokens, positions):
    layer, eps, alpha = cfg["layers"][i], cfg["norm"]["eps"], cfg["postln_alpha"]
    lw = _sub(w, f"l{i}.")
    if layer["type"] != "parallel":
        raise ValueError(layer["type"])
    y = parallel_mixer(x, _sub(lw, "mix."), layer["mixer"], eps, positions)
    x = layer_norm(alpha * x + y, lw["norm1"], lw["norm1.b"], eps)
    mlp = layer.get("mlp")
    if mlp is not None:
        mw = _sub(lw, "mlp.")
        y = dense_ff(x, mw) if mlp["kind"] == "dense" else table_moe(x, mw, mlp, tokens)
        x = layer_norm(alpha * x + y, lw["norm2"], lw["norm2.b"], eps)
    elif "norm2" in lw:                                   # no feed-forward, but the second norm is there
        x = layer_norm(alpha * x, lw["norm2"], lw["norm2.b"], eps)
    return x


def forward(cfg, w: Dict[str, torch.Tensor], tokens, streams: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """One whole request: logits [T, vocab].  `streams` collects x after every layer."""
    tokens = torch.as_tensor(list(tokens), dtype=torch.long)
    positions = torch.arange(tokens.numel())
    x = w["embed"][tokens]
    for i in range(len(cfg["layers"])):
        x = layer_forward(cfg, w, i, x, tokens, positions)
        if streams is not None:
            streams.append(x.clone())
    x = layer_norm(x, w["final.norm"], w["final.norm.b"], cfg["norm"]["eps"])
    return x @ w["head"].T
