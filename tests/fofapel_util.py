"""Test material for the Fofapel architecture: small configurations that differ from each other in every
size and option, and a generator of random checkpoints for them (numpy, its own scales: decays that forget
at a visible rate, queries and keys that make the softmax far from uniform, biases and norm weights that
are neither zero nor one)."""
import json
import os

import numpy as np
import torch


def left(heads, kv_heads, dim, window, rot_dims, base=10000.0, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "mask": {"size": window},
         "scale": float(scale if scale is not None else 2.0 * dim ** -0.5)}
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
    return m


def right(heads, dim, rank):
    return {"heads": heads, "dim": dim, "decay_rank": rank}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, limit, shared=None):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}
    if shared:
        m["shared"] = {"ff": shared[0], "limit": shared[1], "gate": shared[2] if len(shared) > 2 else True}
    return m


def layer(l, r, mlp, ls=1.0, rs=1.0, norm2=None):
    out = {"type": "parallel", "mixer": {"left": l, "right": r, "left_scale": ls, "right_scale": rs}, "mlp": mlp}
    if norm2 is not None:
        out["norm2"] = norm2
    return out


def model(width, vocab, layers, alpha, eps=1e-5):
    return {"architecture": "Fofapel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "postln_alpha": alpha,
            "layers": layers}


# experts first; windows, head shapes and rotated dims that differ from layer to layer (three cache groups);
# part of the head rotated, all of it, none of it; one, some and all query heads a kv head; a time mix whose heads
# are no power of two of 4-channel slices (24), wider than the attention's (80) and of a single head; ranks that
# are no multiple of 8; one, two and three experts a token, with a gated shared expert, one without gate, none;
# a layer without feed-forward
MIX_A = model(64, 301, [
    layer(left(4, 2, 16, 24, 8, 1000.0, 0.3), right(2, 24, 5), moe(5, 3, 24, 1.5, (40, 2.5)), 0.8, 1.3),
    layer(left(3, 3, 32, 7, 32, 50000.0, 0.2), right(1, 80, 8), dense(96), 1.2, 0.9),
    layer(left(2, 1, 16, 1000, 0), right(3, 16, 16), None, 1.0, 0.5),
    layer(left(4, 1, 24, 33, 12, 100.0), right(2, 32, 3), moe(3, 1, 16, 2.0), 0.6, 1.0),
], alpha=2.0)

# a window of one token (a token sees itself and the sink), every expert used by every token, a shared expert
# without gate, a layer without feed-forward that keeps its second norm, alpha below one
MIX_B = model(128, 257, [
    layer(left(2, 2, 64, 1, 64, 250.0), right(4, 32, 16), dense(64), 1.0, 1.0),
    layer(left(8, 2, 16, 50, 4, 7000.0, 0.5), right(2, 64, 24), moe(2, 2, 32, 1.0, (16, 3.0, False)), 1.5, 0.7),
    layer(left(4, 4, 32, 16, 16), right(1, 128, 8), None, 0.9, 1.1, norm2=True),
    layer(left(6, 3, 16, 100, 16, 1.0e6, 0.25), right(8, 16, 12), moe(7, 2, 8, 2.5, (24, 0.7)), 1.0, 1.0),
], alpha=0.7, eps=3e-6)

ONLY_DENSE = model(64, 199, [layer(left(3, 1, 16, 20, 16), right(2, 16, 4), dense(48), 1.1, 0.9)], alpha=1.5)
ONLY_MOE = model(64, 199, [layer(left(2, 2, 24, 9, 6), right(3, 24, 9), moe(4, 2, 16, 2.0, (24, 1.5)), 0.7, 1.4)], alpha=3.0)

CONFIGS = {"A": (MIX_A, 16), "B": (MIX_B, 8), "dense": (ONLY_DENSE, 4), "moe": (ONLY_MOE, 16)}


def random_config(seed):
    """A configuration drawn at random: width, vocabulary, two to four layers that each draw their own head
    counts and sizes, window, rotated dims, time-mix shape, rank and feed-forward."""
    import random
    rng = random.Random(seed)
    width = rng.choice([64, 96, 128, 192, 256])
    vocab = rng.randrange(90, 700)
    layers = []
    for _ in range(rng.randrange(2, 5)):
        dim = rng.choice([16, 24, 32, 48, 64, 80, 128])
        kv = rng.choice([1, 2, 3])
        heads = kv * rng.choice([1, 2, 3, 4])
        while heads * dim % 8:
            heads += kv
        rot = rng.choice([0, dim, dim // 2 // 2 * 2, 2])
        a = left(heads, kv, dim, rng.choice([1, 2, 5, 16, 31, 64, 100, 5000]), rot, rng.choice([100.0, 10000.0, 250000.0]),
                 rng.choice([dim ** -0.5, 2.0 * dim ** -0.5, 4.0 / dim]))       # typical scores of a few units
        td = rng.choice([8, 16, 24, 32, 40, 64, 96, 128])
        th = rng.randrange(1, 5)
        while th * td % 8:
            th += 1
        t = right(th, td, rng.choice([1, 4, 8, 13, 32]))
        kind = rng.choice(["dense", "moe", "moe", "none"])
        if kind == "dense":
            mlp = dense(8 * rng.randrange(1, 40))
        elif kind == "moe":
            e = rng.randrange(1, 10)
            shared = rng.choice([None, (8 * rng.randrange(1, 12), rng.uniform(0.5, 4.0), rng.random() < 0.7)])
            mlp = moe(e, rng.randrange(1, e + 1), 8 * rng.randrange(1, 12), rng.uniform(0.5, 4.0), shared)
        else:
            mlp = None
        layers.append(layer(a, t, mlp, rng.uniform(0.3, 1.6), rng.uniform(0.3, 1.6),
                            norm2=(rng.random() < 0.5) if mlp is None else None))
    return model(width, vocab, layers, alpha=rng.choice([0.5, 1.0, 2.5, 4.0]), eps=rng.choice([1e-5, 1e-6, 1e-4]))


def random_weights(cfg, seed=0, sharpen=3.0):
    """{name: tensor} (float32; the experts' table int32).  `sharpen`: the gain of the projections that make
    scores, gates and decays (3: far from uniform, a misplaced key or a lost state moves the logits; 1: tame, so
    that bfloat16 rounding is not amplified)."""
    lively = 2.0 if sharpen > 1.0 else 1.0
    rng = np.random.default_rng(seed)
    W, V, out = cfg["width"], cfg["vocab"], {}

    def mat(name, rows, cols, gain=1.0):
        out[name] = rng.standard_normal((rows, cols)) * gain / np.sqrt(cols)

    def vec(name, n, mean=0.0, std=0.1):
        out[name] = mean + std * rng.standard_normal(n)

    def glu(p, F):
        mat(p + "gate", F, W, gain=lively)
        mat(p + "up", F, W, gain=lively)
        mat(p + "down", W, F)

    mat("embed", V, W, gain=np.sqrt(W))
    for i, l in enumerate(cfg["layers"]):
        p, a, t = f"l{i}.", l["mixer"]["left"], l["mixer"]["right"]
        vec(p + "norm1", W, 1.0, 0.2)
        vec(p + "norm1.b", W, 0.0, 0.2)
        H, G, D = a["heads"], a["kv_heads"], a["dim"]
        mat(p + "mix.left.q", H * D, W, gain=sharpen)
        vec(p + "mix.left.q.b", H * D, 0.0, 0.3)
        mat(p + "mix.left.k", G * D, W, gain=sharpen)
        vec(p + "mix.left.k.b", G * D, 0.0, 0.3)
        mat(p + "mix.left.g", H, W, gain=lively)
        mat(p + "mix.left.o", W, H * D)
        S, R = t["heads"] * t["dim"], t["decay_rank"]
        for s in "rkvgw":
            out[p + f"mix.right.mu.{s}"] = rng.uniform(0.0, 1.0, W)
        for s in "rkvg":
            mat(p + f"mix.right.{s}", S, W, gain=lively)
        mat(p + "mix.right.w1", R, W, gain=lively)
        mat(p + "mix.right.w2", S, R, gain=lively)
        out[p + "mix.right.w0"] = rng.uniform(-3.0, 0.0, S)
        out[p + "mix.right.u"] = 0.5 * rng.standard_normal((t["heads"], t["dim"]))
        vec(p + "mix.right.norm", S, 1.0, 0.2)
        mat(p + "mix.right.o", W, S)
        mlp = l["mlp"]
        if mlp is not None and mlp["kind"] == "dense":
            glu(p + "mlp.", mlp["ff"])
        elif mlp is not None:
            E, top = mlp["router"]["experts"], mlp["router"]["top"]
            for e in range(E):
                glu(p + f"mlp.e{e}.", mlp["expert"]["ff"])
            out[p + "mlp.table"] = np.stack([rng.permutation(E)[:top] for _ in range(V)]).astype(np.int32)
            if mlp.get("shared"):
                glu(p + "mlp.shared.", mlp["shared"]["ff"])
                if mlp["shared"].get("gate", True):
                    mat(p + "mlp.shared.sg", 1, W, gain=lively)
        if mlp is not None or l.get("norm2"):
            vec(p + "norm2", W, 1.0, 0.2)
            vec(p + "norm2.b", W, 0.0, 0.2)
    vec("final.norm", W, 1.0, 0.2)
    vec("final.norm.b", W, 0.0, 0.2)
    mat("head", V, W, gain=lively)
    return {k: torch.from_numpy(np.asarray(v, dtype=np.int32 if k.endswith(".table") else np.float32))
            for k, v in out.items()}


def make_folder(path, cfg, seed=0, store=torch.float32, sharpen=3.0):
    """config.json and model.safetensors (written with the safetensors library).  Returns (folder, weights).
    The written config.json has no `decay_rank`, `norm2` or `gate`: a loaded model takes them from the tensors."""
    from safetensors.torch import save_file
    folder = str(path)
    os.makedirs(folder, exist_ok=True)
    w = random_weights(cfg, seed, sharpen)
    stripped = json.loads(json.dumps(cfg))
    for l in stripped["layers"]:
        l.pop("norm2", None)
        l["mixer"]["right"].pop("decay_rank", None)
        if l["mlp"] and l["mlp"].get("shared"):
            l["mlp"]["shared"].pop("gate", None)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(stripped, f)
    save_file({k: (v if v.dtype == torch.int32 else v.to(store)).contiguous() for k, v in w.items()},
              os.path.join(folder, "model.safetensors"))
    return folder, w


def rounded(weights, dtype=torch.bfloat16):
    """The weights as a bfloat16 engine holds them: everything rounded, as float64 (tables stay integers)."""
    return {k: (v if v.dtype == torch.int32 else v.to(dtype).to(torch.float64)) for k, v in weights.items()}


def as_double(weights):
    return {k: (v if v.dtype == torch.int32 else v.double()) for k, v in weights.items()}


def row_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    """Root mean square of the difference of two rows of logits (means taken off) over the
    reference row's own root mean square."""
    d = got.double().cpu() - ref.double().cpu()
    d = d - d.mean()
    r = ref.double().cpu() - ref.double().cpu().mean()
    return float(torch.sqrt((d * d).mean()) / torch.sqrt((r * r).mean()).clamp_min(1e-30))
