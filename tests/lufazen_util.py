"""Test material for the Lufazen architecture: small configurations that differ from each other
in every size and option, and a generator of random checkpoints for them (numpy, its own scales:
norm weights around zero, decays that forget at a visible rate, sharpened attention)."""
import json
import os

import numpy as np
import torch

YARN = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale=None, base=10000.0, scaling=None, kv_from=None, dims=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "scale": float(scale if scale is not None else (dim + rot_dim) ** -0.5)}
    if rot_dim:
        m["rot"] = {"base": base, "dims": dims or rot_dim}
        if scaling:
            m["rot"]["scaling"] = dict(scaling)
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def delta(heads, kv_heads, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def layer(kind, mixer, ff=None, limit=3.0):
    return {"type": kind, "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff, "limit": limit}}


def model(width, vocab, layers, eps=1e-5, softcap=20.0):
    cfg = {"architecture": "Lufazen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if softcap:
        cfg["logit_softcap"] = softcap
    return cfg


# recurrent layers around two attention layers, the second of which reads the first one's cache;
# grouped q/k heads, dim != vdim, three and two taps, a layer without feed-forward
MIX_A = model(64, 301, [
    layer("channel_delta", delta(4, 2, 16, 24, 3), ff=96),
    layer("latent_attention", latent(3, 24, 8, 16, 40, 48, scaling=YARN), ff=80, limit=1.5),
    layer("latent_attention", latent(2, 16, 8, 32, 24, 48, scaling=YARN, kv_from=1), ff=96),
    layer("channel_delta", delta(2, 2, 32, 16, 2)),
])
RANKS_A = {0: (12, 20), 3: (8, 4)}

# attention first; two attention layers with caches of different shapes (two cache groups); no
# scaling of the rotation in one, fewer rotated dims than the key part has in the other; no soft cap
MIX_B = model(128, 257, [
    layer("latent_attention", latent(4, 32, 16, 32, 64, 64, base=500.0), ff=192),
    layer("channel_delta", delta(6, 2, 64, 64, 4), ff=128, limit=2.5),
    layer("latent_attention", latent(2, 64, 32, 24, 32, 96, base=50000.0, scaling={"factor": 3.0, "original": 40,
                                                                                  "fast": 8.0, "slow": 1.0}, dims=16)),
    layer("channel_delta", delta(1, 1, 8, 40, 5), ff=64),
], eps=3e-6, softcap=0.0)
RANKS_B = {1: (16, 16), 3: (5, 3)}

ONLY_LATENT = model(64, 199, [layer("latent_attention", latent(2, 16, 16, 24, 32, 40, scaling=YARN))])
ONLY_DELTA = model(64, 199, [layer("channel_delta", delta(3, 1, 24, 16, 4))])
RANKS_ONLY = {0: (10, 6)}

CONFIGS = {"A": (MIX_A, RANKS_A, 16), "B": (MIX_B, RANKS_B, 8), "latent": (ONLY_LATENT, {}, 4),
           "delta": (ONLY_DELTA, RANKS_ONLY, 16)}


def random_weights(cfg, ranks, seed=0, sharpen=3.0):
    """{name: float32 tensor}.  `ranks`: {layer: (rank of a1, rank of g1)} for the recurrent layers.
    `sharpen`: the gain of the projections that make scores, gates and decays (3: far from uniform, a
    misplaced key or a lost state moves the logits; 1: tame, so that bfloat16 rounding is not amplified)."""
    lively = 2.0 if sharpen > 1.0 else 1.0
    rng = np.random.default_rng(seed)
    W, out = cfg["width"], {}

    def mat(name, rows, cols, gain=1.0):
        out[name] = rng.standard_normal((rows, cols)) * gain / np.sqrt(cols)

    def vec(name, n, mean=0.0, std=0.1):
        out[name] = mean + std * rng.standard_normal(n)

    mat("embed", cfg["vocab"], W, gain=np.sqrt(W))
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        vec(p + "norm1", W)
        vec(p + "ls1", W, 0.7, 0.2)
        if l["type"] == "latent_attention":
            H, D, R, V = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            mat(p + "mix.dq", m["q_rank"], W)
            vec(p + "mix.dq.norm", m["q_rank"], 1.0)
            mat(p + "mix.uq", H * (D + R), m["q_rank"], gain=sharpen)
            if m.get("kv_from") is None:
                mat(p + "mix.dkv", m["kv_rank"] + R, W, gain=sharpen)
                vec(p + "mix.dkv.norm", m["kv_rank"], 1.0)
            mat(p + "mix.uk", H * D, m["kv_rank"])
            mat(p + "mix.uv", H * V, m["kv_rank"])
            mat(p + "mix.g", H, W, gain=lively)
            mat(p + "mix.o", W, H * V)
        else:
            H, KH, D, V, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            ra, rg = ranks[i]
            for n, rows in (("q", KH * D), ("k", KH * D), ("v", H * V)):
                mat(p + f"mix.{n}", rows, W, gain=lively)
                out[p + f"mix.{n}.conv"] = rng.standard_normal((rows, taps)) * 0.6
            mat(p + "mix.b", H, W, gain=lively)
            out[p + "mix.A_log"] = rng.uniform(-1.5, 0.5, H)
            vec(p + "mix.norm", V, 1.0)
            mat(p + "mix.a1", ra, W)
            mat(p + "mix.a2", H * D, ra, gain=lively)
            vec(p + "mix.dt_bias", H * D, -1.0, 1.0)
            mat(p + "mix.g1", rg, W)
            mat(p + "mix.g2", H * V, rg, gain=lively)
            mat(p + "mix.o", W, H * V)
        if l["mlp"] is not None:
            F = l["mlp"]["ff"]
            mat(p + "mlp.gate", F, W, gain=lively)
            mat(p + "mlp.up", F, W, gain=lively)
            mat(p + "mlp.down", W, F)
            vec(p + "norm2", W)
            vec(p + "ls2", W, 0.7, 0.2)
    vec("final.norm", W)
    mat("head", cfg["vocab"], W, gain=lively)
    return {k: torch.from_numpy(np.asarray(v, dtype=np.float32)) for k, v in out.items()}


def make_folder(path, cfg, ranks, seed=0, store=torch.float32, sharpen=3.0):
    """config.json and model.safetensors (written with the safetensors library).  Returns (folder, weights)."""
    from safetensors.torch import save_file
    folder = str(path)
    os.makedirs(folder, exist_ok=True)
    w = random_weights(cfg, ranks, seed, sharpen)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(store).contiguous() for k, v in w.items()}, os.path.join(folder, "model.safetensors"))
    return folder, w


def rounded(weights, dtype=torch.bfloat16):
    """The weights as a bfloat16 engine holds them: everything rounded, as float64."""
    return {k: v.to(dtype).to(torch.float64) for k, v in weights.items()}


def row_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    """Root mean square of the difference of two rows of logits (means taken off) over the
    reference row's own root mean square."""
    d = got.double().cpu() - ref.double().cpu()
    d = d - d.mean()
    r = ref.double().cpu() - ref.double().cpu().mean()
    return float(torch.sqrt((d * d).mean()) / torch.sqrt((r * r).mean()).clamp_min(1e-30))
