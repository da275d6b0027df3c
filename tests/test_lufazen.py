"""The Lufazen architecture without a GPU: its configuration reader, the model as data, the
checkpoint's names, the rotation's frequencies against the plain implementation, and the plain
implementation against itself (properties that a wrong reading of the equations breaks)."""
import copy

import pytest
import torch

import plain_lufazen as plain
from lufazen_util import CONFIGS, MIX_A, MIX_B, RANKS_A, RANKS_B, random_weights


def _shapes(cfg, ranks):
    return {k: tuple(v.shape) for k, v in random_weights(cfg, ranks).items()}


@pytest.mark.parametrize("name", ["A", "B", "latent", "delta"])
def test_spec_declares_exactly_the_checkpoints_tensors(name):
    from tiny_llm_amd.config import resolve
    from tiny_llm_amd.models.decoder import Decoder
    cfg, ranks, _ = CONFIGS[name]
    shapes = _shapes(cfg, ranks)
    typed, spec = resolve(cfg, shapes)
    dec = Decoder(spec, dtype="float32", device="cpu")
    declared = {s.name: tuple(s.shape) for s in dec.weight_specs()}
    assert declared == shapes
    assert len(spec.plan) == len(cfg["layers"])


def test_ranks_come_from_tensor_shapes_or_from_the_configuration():
    from tiny_llm_amd.config import ConfigError, resolve
    typed, _ = resolve(MIX_A, _shapes(MIX_A, RANKS_A))
    assert (typed.layers[0].mixer.decay_rank, typed.layers[0].mixer.gate_rank) == RANKS_A[0]
    assert (typed.layers[3].mixer.decay_rank, typed.layers[3].mixer.gate_rank) == RANKS_A[3]
    with pytest.raises(ConfigError):
        resolve(MIX_A)                              # neither shapes nor keys
    by_hand = copy.deepcopy(MIX_A)
    for i, (ra, rg) in RANKS_A.items():
        by_hand["layers"][i]["mixer"].update(decay_rank=ra, gate_rank=rg)
    assert resolve(by_hand)[0] == typed


def test_plan_and_cache_groups():
    from tiny_llm_amd.config import resolve
    from tiny_llm_amd.models.decoder import Decoder
    _, spec = resolve(MIX_A, _shapes(MIX_A, RANKS_A))
    assert [e.cache_of for e in spec.plan] == [None, None, 1, None]
    dec = Decoder(spec, dtype="float32", device="cpu")
    assert list(dec.cache_specs()) == [(1, "mixer")]
    assert dec.cache_readers() == {(2, "mixer"): (1, "mixer")}
    assert sorted(dec.state_specs()) == [(0, "mixer"), (3, "mixer")]
    assert "ffn" not in dec.layers[3].by_role            # a layer without feed-forward
    # two attention layers with caches of different shapes: two groups, each with its own pages
    from tiny_llm_amd.cache import CacheManager
    _, spec_b = resolve(MIX_B, _shapes(MIX_B, RANKS_B))
    dec_b = Decoder(spec_b, dtype="float32", device="cpu")
    cm = CacheManager(dec_b.cache_specs(), dec_b.state_specs(), 8, 10, 2)
    assert len(cm.groups) == 2


def test_refusals():
    from tiny_llm_amd.config import ConfigError, resolve
    shapes = _shapes(MIX_A, RANKS_A)

    def broken(change):
        c = copy.deepcopy(MIX_A)
        change(c)
        with pytest.raises((ConfigError, ValueError)):
            resolve(c, shapes)

    broken(lambda c: c["layers"][0].update(type="unknown_mixer"))
    broken(lambda c: c["layers"][2]["mixer"].update(kv_from=0))         # not an attention layer
    broken(lambda c: c["layers"][2]["mixer"].update(kv_from=2))         # not an earlier layer
    broken(lambda c: c["layers"][2]["mixer"].update(kv_rank=56))        # differs from the cache it reads
    broken(lambda c: c["layers"][1]["mlp"].update(kind="routed"))
    broken(lambda c: c["layers"][0]["mixer"].update(kv_heads=3))
    broken(lambda c: c.pop("norm"))
    chained = copy.deepcopy(MIX_A)
    chained["layers"].append(copy.deepcopy(chained["layers"][2]))
    chained["layers"][4]["mixer"]["kv_from"] = 2                           # reads a layer that has no cache of its own
    with pytest.raises((ConfigError, ValueError)):
        resolve(chained, shapes)


@pytest.mark.parametrize("dims,base,scaling", [
    (16, 500000.0, {"factor": 4.0, "original": 1024, "fast": 32.0, "slow": 1.0}),
    (8, 10000.0, {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}),
    (32, 50000.0, {"factor": 3.0, "original": 40, "fast": 8.0, "slow": 1.0}),
    (64, 10000.0, {"factor": 40.0, "original": 4096, "fast": 32.0, "slow": 1.0}),
    (16, 500.0, None),
])
def test_angle_tables_against_the_plain_rotation(dims, base, scaling):
    """The rotary part's tables (host float64, rounded once) equal cos and sin of the plain
    implementation's frequencies, magnitude included; some frequencies are kept, some divided."""
    from tiny_llm_amd.parts.rotary import RotaryEmbedding
    part = RotaryEmbedding("p", torch.float32, "cpu", head_dim=dims, theta=base, max_position=300,
                           scaling=dict(scaling, kind="yarn") if scaling else None)
    f, mag = plain.yarn_frequencies(dims, base, scaling)
    pos = torch.arange(300, dtype=torch.float64)
    assert torch.allclose(part.cos.double(), torch.cos(pos[:, None] * f) * mag, atol=1e-6)
    assert torch.allclose(part.sin.double(), torch.sin(pos[:, None] * f) * mag, atol=1e-6)
    if scaling:
        plain_f = base ** (-2.0 * torch.arange(dims // 2, dtype=torch.float64) / dims)
        assert torch.isclose(f[0], plain_f[0]) or scaling["factor"] > 1           # sanity of the blend's ends
        assert torch.all(f <= plain_f * (1 + 1e-12)) and torch.all(f >= plain_f / scaling["factor"] * (1 - 1e-12))


def test_plain_delta_rule_is_causal_and_forgets():
    """Changing a late token leaves earlier outputs alone; with the decay forced to zero the state
    holds the current token only, so the output is beta * (q . k) * v."""
    g = torch.Generator().manual_seed(1)
    m = {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 6, "conv": 3}
    W = 16
    w = {k: v.double() for k, v in random_weights(
        {"vocab": 11, "width": W, "norm": {"eps": 1e-5}, "layers": [{"type": "channel_delta", "mixer": m, "mlp": None}]},
        {0: (4, 4)}, seed=2).items()}
    mw = plain.sub(w, "l0.mix.")
    h = torch.randn(12, W, generator=g, dtype=torch.float64)
    y = plain.channel_delta(h, mw, m, 1e-5)
    h2 = h.clone()
    h2[9] += 1.0
    y2 = plain.channel_delta(h2, mw, m, 1e-5)
    assert torch.allclose(y[:9], y2[:9]) and not torch.allclose(y[9:], y2[9:])
    forget = dict(mw)
    forget["A_log"] = torch.full_like(mw["A_log"], 20.0)           # decay exp(-e^20 * softplus) = 0
    y3 = plain.channel_delta(h, forget, m, 1e-5)
    assert torch.isfinite(y3).all()


def test_plain_latent_attention_sees_only_the_past():
    g = torch.Generator().manual_seed(4)
    cfg, ranks, _ = CONFIGS["latent"]
    w = {k: v.double() for k, v in random_weights(cfg, ranks, seed=3).items()}
    a = plain.forward(cfg, w, [5, 9, 3, 100, 42, 7])
    b = plain.forward(cfg, w, [5, 9, 3, 100, 1, 7])
    assert torch.allclose(a[:4], b[:4]) and not torch.allclose(a[4:], b[4:])
