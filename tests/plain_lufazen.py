"""A plain, slow Lufazen: every mechanism of the design as one small function, written from its
equations with torch on the CPU (float64 unless told otherwise).  It shares no code with the
engine: it reads config.json's own keys and the checkpoint's tensor names, keeps whole sequences
(no cache, no pages, no state slots) and runs one request at a time.

Notation: x [T, W] is the residual stream, h a sublayer's input (x itself: the norms of this
design sit on the sublayers' outputs), weights are [out, in] and applied as h @ W.T.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm_around_zero(x, w, eps):
    """The layer norms and the final norm: the stored weight is the distance from one."""
    return rms_unit(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    """The norms inside the mixers: the stored weight is the factor itself."""
    return rms_unit(x, eps) * w


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# ------------------------------------------------------------------------ rotation
def yarn_frequencies(dims: int, base: float, scaling: Optional[dict]):
    """(f [dims/2], magnitude): f_i = base^(-2i/dims), blended towards f_i / factor for the slow
    dimensions; cos and sin are multiplied by `magnitude`."""
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def dim_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(scaling["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    f = f / factor * ramp + f * (1.0 - ramp)
    return f, 0.1 * math.log(factor) + 1.0


def rotate_half(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float, scaling) -> torch.Tensor:
    """x [T, ..., D]: the first `dims` of the last axis rotate, i paired with i + dims/2."""
    f, mag = yarn_frequencies(dims, base, scaling)
    a = positions.to(torch.float64)[:, None] * f[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    cos, sin = (torch.cos(a) * mag).reshape(shape).to(x.dtype), (torch.sin(a) * mag).reshape(shape).to(x.dtype)
    u, v = x[..., :dims // 2], x[..., dims // 2:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


# ---------------------------------------------------------------- latent attention
def latent_kv(h, w, m, eps, positions):
    """What a layer with a W_dkv of its own keeps per token: (latent c [T, kv_rank],
    rotated shared key part [T, rot_dim])."""
    r = m["kv_rank"]
    d = h @ w["dkv"].T
    c = norm_plain(d[:, :r], w["dkv.norm"], eps)
    kr = rotate_half(d[:, r:], positions, m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    return c, kr


def latent_attention(h, w, m, eps, positions, kv):
    """h [T, W] -> [T, W].  `kv` = (c, kr) of this layer or of the layer it borrows from."""
    T = h.shape[0]
    H, D, R, V = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    c, kr = kv
    cq = norm_plain(h @ w["dq"].T, w["dq.norm"], eps)
    q = (cq @ w["uq"].T).reshape(T, H, D + R)
    q_plain = q[..., :D]
    q_rot = rotate_half(q[..., D:], positions, m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    k_plain = (c @ w["uk"].T).reshape(T, H, D)
    v = (c @ w["uv"].T).reshape(T, H, V)
    s = torch.einsum("thd,jhd->htj", q_plain, k_plain) + torch.einsum("thr,jr->htj", q_rot, kr)
    s = s * m["scale"]
    causal = positions[None, :] <= positions[:, None]
    s = s.masked_fill(~causal[None], float("-inf"))
    p = torch.softmax(s, dim=-1)
    o = torch.einsum("htj,jhv->thv", p, v)
    gate = torch.sigmoid(h @ w["g"].T)
    o = o * gate[:, :, None]
    return o.reshape(T, H * V) @ w["o"].T


# -------------------------------------------------------------------- delta rule
def causal_conv_silu(x, taps_w):
    """x [T, C], taps_w [C, taps] (last column the current token's), zeros before the start."""
    T, C = x.shape
    taps = taps_w.shape[1]
    xp = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x], dim=0)
    y = torch.zeros_like(x)
    for j in range(taps):
        y = y + xp[j:j + T] * taps_w[:, j][None, :]
    return y * torch.sigmoid(y)


def channel_delta(h, w, m, eps):
    """Gated delta rule with one decay per head and key channel.  h [T, W] -> [T, W]."""
    T = h.shape[0]
    H, KH, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = causal_conv_silu(h @ w["q"].T, w["q.conv"]).reshape(T, KH, D)
    k = causal_conv_silu(h @ w["k"].T, w["k.conv"]).reshape(T, KH, D)
    v = causal_conv_silu(h @ w["v"].T, w["v.conv"]).reshape(T, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w["b"].T)                                      # [T, H]
    a = (h @ w["a1"].T) @ w["a2"].T + w["dt_bias"]                          # [T, H * D]
    decay = torch.exp(-torch.exp(w["A_log"])[None, :, None] * softplus(a).reshape(T, H, D))
    rep = H // KH
    S = torch.zeros(H, D, V, dtype=h.dtype)
    o = torch.zeros(T, H, V, dtype=h.dtype)
    for t in range(T):
        for hd in range(H):
            kt, qt = k[t, hd // rep], q[t, hd // rep]
            S[hd] = decay[t, hd][:, None] * S[hd]
            u = beta[t, hd] * (v[t, hd] - S[hd].T @ kt)
            S[hd] = S[hd] + kt[:, None] * u[None, :]
            o[t, hd] = S[hd].T @ qt
    o = rms_unit(o, eps) * w["norm"][None, None, :]
    gate = torch.sigmoid((h @ w["g1"].T) @ w["g2"].T).reshape(T, H, V)
    return (o * gate).reshape(T, H * V) @ w["o"].T


# ----------------------------------------------------------------- feed-forward
def dense_ff(h, w, mlp):
    lim = float(mlp["limit"])
    g = torch.clamp(h @ w["gate"].T, max=lim)
    u = torch.clamp(h @ w["up"].T, -lim, lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w["down"].T


# ------------------------------------------------------------------------ model
def sub(weights: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(config: dict, weights: Dict[str, torch.Tensor], tokens, dtype=torch.float64, layers_out: List = None):
    """Logits [T, vocab] of one whole sequence.  `layers_out` (a list) receives the residual stream
    after every layer."""
    W = {k: v.to(dtype) for k, v in weights.items()}
    eps = float(config["norm"]["eps"])
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    T = tokens.numel()
    positions = torch.arange(T)
    x = W["embed"][tokens]
    kept = {}
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        mw = sub(W, p + "mix.")
        if layer["type"] == "latent_attention":
            if m.get("kv_from") is None:
                kept[i] = latent_kv(x, mw, m, eps, positions)
                kv = kept[i]
            else:
                kv = kept[int(m["kv_from"])]
            y = latent_attention(x, mw, m, eps, positions, kv)
        elif layer["type"] == "channel_delta":
            y = channel_delta(x, mw, m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + norm_around_zero(y, W[p + "norm1"], eps) * W[p + "ls1"]
        if layer.get("mlp") is not None:
            y = dense_ff(x, sub(W, p + "mlp."), layer["mlp"])
            x = x + norm_around_zero(y, W[p + "norm2"], eps) * W[p + "ls2"]
        if layers_out is not None:
            layers_out.append(x.clone())
    x = norm_around_zero(x, W["final.norm"], eps)
    logits = x @ W["head"].T
    cap = config.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return logits
