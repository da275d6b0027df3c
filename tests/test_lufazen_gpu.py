"""The Lufazen architecture in the engine against the plain implementation of its equations
(tests/plain_lufazen.py): each mechanism alone, every way of cutting the work, pages and state slots
used again, captured steps, long decoding, generation through the entry point, and keys that a
crafted query singles out at the places where an index can be off by one."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_lufazen as plain
import traces
from lufazen_util import CONFIGS, make_folder, rounded, row_err
from util import random_tokens

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# float32: everything is computed in 32 bits, what is left is the order of sums.  bfloat16: weights are
# rounded for the plain model too; the products' inputs and outputs are rounded in the engine only, and
# the models are made without the sharpening of the attention that would amplify that rounding.  A fault of
# a mechanism (a key off by one, a state lost, a wrong slot) moves a row by its whole size in either
# precision; the float32 runs are the sharp test, the bfloat16 runs cover that path's own kernels,
# strides and alignments.  A row's error is the same in every cutting, to the digit: it is rounding.
TOL = {"float32": 2e-4, "bfloat16": 1e-1}
LENGTHS = {"A": [70, 133, 33, 200, 97, 64], "B": [1, 9, 40, 100, 150, 57], "latent": [40, 75, 130, 9],
           "delta": [24, 121, 48, 5]}

_cache = {}


def material(name, dtype, tmp_path_factory):
    key = (name, dtype)
    if key not in _cache:
        cfg, ranks, block = CONFIGS[name]
        folder, w = make_folder(tmp_path_factory.mktemp(f"lufazen_{name}_{dtype}"), cfg, ranks, seed=11,
                                store=torch.bfloat16 if dtype == "bfloat16" else torch.float32,
                                sharpen=1.0 if dtype == "bfloat16" else 3.0)
        w64 = rounded(w) if dtype == "bfloat16" else {k: v.double() for k, v in w.items()}
        reqs = {f"r{i}": random_tokens(n, cfg["vocab"], 100 * i + len(name)) for i, n in enumerate(LENGTHS[name])}
        ref = {rid: plain.forward(cfg, w64, toks) for rid, toks in reqs.items()}
        _cache[key] = (folder, cfg, w64, reqs, ref, block)
    return _cache[key]


def make_runner(folder, dtype, block_size, max_tokens, max_seqs=4):
    from tiny_llm_amd.config import EngineConfig
    from tiny_llm_amd.engine.loading import build_runner, load_model
    engine = EngineConfig(dtype=dtype, kv_block_size=block_size, max_cache_tokens=max_tokens, max_num_seqs=max_seqs,
                          max_num_batched_tokens=1 << 16, use_graphs=False)
    _, dec = load_model(folder, engine)
    runner = build_runner(dec, engine)
    for g in runner.cache.groups:               # stale or unwritten pages must never reach a result
        for t in g.tensors.values():
            t.fill_(float("nan"))
    for st in runner.cache.states.values():     # a state slot is cleared when a request takes it
        st.fill_(float("nan"))
    return runner


def replay(runner, steps, use_graph=False):
    from tiny_llm_amd.engine.step import StepEntry
    out = {}
    for s in steps:
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]], use_graph=use_graph)
        if logits.shape[0]:
            out[s["step"]] = logits.cpu()
        for rid in s["end"]:
            runner.finish(rid)
        runner.cache.audit()
    return out


def check(out, steps, ref, tol):
    rows = traces.rows_of(steps)
    assert set(rows) == set(out)
    worst = 0.0
    for step, where in rows.items():
        got = out[step]
        assert got.shape[0] == len(where)
        for i, (rid, pos) in enumerate(where):
            assert torch.isfinite(got[i]).all(), (step, rid, pos)
            e = row_err(got[i], ref[rid][pos])
            worst = max(worst, e)
            assert e < tol, f"step {step}: request {rid} position {pos}: err {e:.3e}"
    return worst


def r64(n):
    return -(-n // 64) * 64


def all_free(runner):
    return runner.cache.free_blocks() == [g.pool.num_blocks for g in runner.cache.groups] and \
        runner.cache.free_slots == runner.cache.max_seqs


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["latent", "delta", "A", "B"])
def test_whole_tail_portions(name, dtype, tmp_path_factory):
    """Each request alone: whole, its tail token by token, and in portions down to two tokens (one-layer
    models of each mixer alone, then the two mixed models)."""
    folder, cfg, w, reqs, ref, block = material(name, dtype, tmp_path_factory)
    biggest = max(r64(len(t)) for t in reqs.values())
    for build in (traces.whole, traces.tail_one_by_one, traces.portions):
        steps = build(reqs)
        runner = make_runner(folder, dtype, block, biggest, max_seqs=1)
        worst = check(replay(runner, steps), steps, ref, TOL[dtype])
        print(f"{name} {dtype} {build.__name__}: worst {worst:.2e}")
        assert all_free(runner)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_mixed_batches_reuse_pages_and_slots(name, dtype, tmp_path_factory):
    """Up to four live requests of unequal length in one step, six requests through four state slots
    and a pool smaller than their sum; every row against the request run alone by the plain model."""
    folder, cfg, w, reqs, ref, block = material(name, dtype, tmp_path_factory)
    for seed in (0, 1):
        steps, peak = traces.mixed(reqs, seed=seed)
        assert peak < sum(r64(len(t)) for t in reqs.values())
        runner = make_runner(folder, dtype, block, peak, max_seqs=4)
        worst = check(replay(runner, steps), steps, ref, TOL[dtype])
        print(f"{name} {dtype} mixed {seed}: worst {worst:.2e}, pool {peak}")
        assert all_free(runner)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_steps(dtype, tmp_path_factory):
    """The same cuttings with every step as a HIP graph of its shape (padding tokens, requests and
    rows), twice over so that the second pass replays what the first captured."""
    folder, cfg, w, reqs, ref, block = material("A", dtype, tmp_path_factory)
    steps, peak = traces.mixed(reqs, seed=2)
    runner = make_runner(folder, dtype, block, max(peak, max(r64(len(t)) for t in reqs.values())))
    for st in (steps, traces.portions(reqs), traces.tail_one_by_one(reqs)):
        for again in range(2):
            check(replay(runner, st, use_graph=True), st, ref, TOL[dtype])
            assert all_free(runner)
    assert runner.graph_steps > runner.eager_steps
    assert not any(g.capture_failed for g in runner._graphs.values())
    assert runner.decoder.graph_safe


def test_first_tokens(tmp_path_factory):
    folder, cfg, w, reqs, ref, block = material("A", "float32", tmp_path_factory)
    runner = make_runner(folder, "float32", block, 64)
    from tiny_llm_amd.engine.step import StepEntry
    for n in (1, 2, 3, 4):
        logits = runner.step([StepEntry("x", reqs["r3"][:n], list(range(n)))]).cpu()
        runner.finish("x")
        for i in range(n):
            assert row_err(logits[i], ref["r3"][i]) < TOL["float32"]


def test_long_decoding(tmp_path_factory):
    """Several hundred single-token steps: the recurrent state is carried that far, every page
    edge is crossed, and the rotation passes the length its scaling calls the original one."""
    folder, cfg, w, reqs, ref, block = material("A", "float32", tmp_path_factory)
    toks = random_tokens(330, cfg["vocab"], 4242)
    want = plain.forward(cfg, w, toks)
    runner = make_runner(folder, "float32", block, r64(330))
    from tiny_llm_amd.engine.step import StepEntry
    got = [runner.step([StepEntry("long", toks[:6], list(range(6)))]).cpu()]
    for i in range(6, 330):
        got.append(runner.step([StepEntry("long", [toks[i]], [0])]).cpu())
    got = torch.cat(got)
    worst = max(row_err(got[i], want[i]) for i in range(330))
    print(f"long decoding: worst {worst:.2e}")
    assert worst < TOL["float32"]


@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_the_engine(graphs, tmp_path_factory):
    """Engine.generate (scheduler, portions, captured steps, runs of chained decode steps) against
    greedy decoding with the plain model."""
    folder, cfg, w, reqs, ref, block = material("B", "float32", tmp_path_factory)
    from tiny_llm_amd import Engine, SamplingParams
    prompts = [reqs["r2"][:21], reqs["r3"][:5], reqs["r4"][:34]]
    eng = Engine(folder, dtype="float32", kv_block_size=block, max_num_seqs=2, max_num_batched_tokens=24,
                 max_model_len=256, use_graphs=graphs)
    out = eng.generate(prompts, SamplingParams.greedy(40, ignore_eos=True))
    for p, o in zip(prompts, out):
        seq = list(p)
        for _ in range(40):
            seq.append(int(plain.forward(cfg, w, seq)[-1].argmax()))
        assert o == seq[len(p):]
    eng.runner.cache.audit()
    if graphs:
        assert eng.runner.graph_steps > 0


def test_trace_run_program(tmp_path_factory, tmp_path):
    folder, cfg, w, reqs, ref, block = material("A", "bfloat16", tmp_path_factory)
    steps, peak = traces.mixed(reqs, seed=3)
    out_dir = tmp_path / "out"
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "bfloat16",
         "--out", str(out_dir), "--max-tokens", str(peak)],
        input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done ")] == [f"done {s['step']}" for s in steps]
    out = {}
    for step, where in traces.rows_of(steps).items():
        arr = np.fromfile(out_dir / f"{step}.f32", dtype="<f4")
        assert arr.size == len(where) * cfg["vocab"]
        out[step] = torch.from_numpy(arr.reshape(len(where), cfg["vocab"]))
    check(out, steps, ref, TOL["bfloat16"])


# ------------------------------------------------------------------ kernels with crafted inputs
def _paged(rows: torch.Tensor, table, block, n_blocks, dtype):
    """rows [n, w] laid into pages [n_blocks, block, w] at the blocks `table` names; NaN elsewhere."""
    pages = torch.full((n_blocks, block, rows.shape[1]), float("nan"), dtype=dtype, device="cuda")
    for j in range(rows.shape[0]):
        pages[table[j // block], j % block] = rows[j].to(dtype)
    return pages


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, "matrix cores", "matrix cores, split keys",
                                   "matrix cores, many rows"])
def test_latent_attention_finds_one_key(dtype):
    """One query per place of interest is aligned with the latent of one key (and scaled so that this
    score stands out): the result must be that key's latent.  Keys at the first positions, at both
    sides of page edges, hundreds of tokens back, the query's own position; and the position behind
    the query, which the mask must hide however large its score is."""
    from tiny_llm_amd.kernels import ops
    flash = isinstance(dtype, str)
    dtype_name = dtype if flash else ""
    splits = 3 if flash and "split" in dtype else 1
    dtype = torch.bfloat16 if flash else dtype
    g = torch.Generator().manual_seed(5)
    # the matrix-core kernels with more heads than one tile of 16 rows holds, and not a multiple of it
    n, kv_rank, rot, block, heads = 700, 48 if flash else 40, 8, 16, 20 if flash else 3
    lat = torch.randn(n, kv_rank, generator=g)
    lat = lat / lat.norm(dim=1, keepdim=True)
    rope = torch.randn(n, rot, generator=g) * 0.1
    table = torch.randperm(64, generator=g)[: -(-n // block)].tolist()
    pages_l, pages_r = _paged(lat, table, block, 64, dtype), _paged(rope, table, block, 64, dtype)
    cases = [(699, 0), (699, 1), (699, 15), (699, 16), (699, 17), (699, 698), (699, 699), (650, 63), (650, 64),
             (31, 31), (32, 31), (16, 15), (0, 0), (300, 300), (300, 1)]
    T = len(cases)
    qa = torch.zeros(T, heads, kv_rank + rot)
    for i, (pos, key) in enumerate(cases):
        for h in range(heads):
            # head 0 aims at the case's key, the others at keys of their own around it
            qa[i, h, :kv_rank] = 60.0 * lat[(key + 7 * h) % (pos + 1)]
            if pos + 1 < n:                       # the key behind the query would win if it were seen
                qa[i, h, :kv_rank] += 90.0 * lat[pos + 1]
    positions = torch.tensor([c[0] for c in cases], dtype=torch.int32, device="cuda")
    bt = torch.tensor([table + [0] * (64 - len(table))], dtype=torch.int32, device="cuda")
    out = torch.empty(T, heads, kv_rank, dtype=dtype, device="cuda")
    if flash and "many" in dtype_name:
        # the kernel of steps with many rows: a tile per query here, each a request of its own
        each = torch.arange(T, dtype=torch.int32, device="cuda")
        ops.latent_prefill(qa.cuda(), pages_l, pages_r, bt.repeat(T, 1).contiguous(),
                           (each, each.clone(), torch.ones_like(each)), positions, out, 1.0)
    elif flash:
        # every query a request of its own (the same pages under every row of the table), as in a decode step
        part = torch.empty(splits * T * heads * (kv_rank + 2), device="cuda") if splits > 1 else None
        ops.latent_flash(qa.cuda(), pages_l, pages_r, bt.repeat(T, 1).contiguous(), None, positions, out, 1.0, None,
                         splits, part)
    else:
        ops.latent_attention(qa.cuda(), pages_l, pages_r, bt, torch.zeros(T, dtype=torch.int32, device="cuda"),
                             positions, out, 1.0)
    # the plain softmax over the visible keys
    lat_r, rope_r = lat.to(dtype).double(), rope.to(dtype).double()
    for i, (pos, key) in enumerate(cases):
        for h in range(heads):
            s = qa[i, h, :kv_rank].double() @ lat_r[:pos + 1].T + qa[i, h, kv_rank:].double() @ rope_r[:pos + 1].T
            want = torch.softmax(s, dim=0) @ lat_r[:pos + 1]
            got = out[i, h].double().cpu()
            assert torch.isfinite(got).all()
            assert (got - want).abs().max() < (2e-5 if dtype == torch.float32 else 1e-2), (pos, key, h)


def test_delta_rule_state_over_slots_and_tiny_portions():
    """The recurrence kernels alone: three requests of unequal length in slots out of order, fed in
    portions of 1 to 7 tokens, against the plain recurrence over each whole sequence; convolution
    inputs saved across portions shorter than the taps."""
    from tiny_llm_amd.kernels import ops
    g = torch.Generator().manual_seed(9)
    H, KH, D, V, taps = 4, 2, 16, 24, 4
    C = 2 * KH * D + H * V
    lens = [23, 9, 40]
    slots = [2, 0, 3]
    w = {"q.conv": torch.randn(KH * D, taps, generator=g) * 0.6, "k.conv": torch.randn(KH * D, taps, generator=g) * 0.6,
         "v.conv": torch.randn(H * V, taps, generator=g) * 0.6, "A_log": torch.rand(H, generator=g) - 1.0,
         "dt_bias": torch.randn(H * D, generator=g) - 1.0}
    p_all = [torch.randn(n, C + H, generator=g) for n in lens]        # [q | k | v | beta's input]
    a_all = [torch.randn(n, H * D, generator=g) for n in lens]
    # plain recurrence, float64
    want = []
    for p, a in zip(p_all, a_all):
        n = p.shape[0]
        pd, ad = p.double(), a.double()
        q = plain.causal_conv_silu(pd[:, :KH * D], w["q.conv"].double()).reshape(n, KH, D)
        k = plain.causal_conv_silu(pd[:, KH * D:2 * KH * D], w["k.conv"].double()).reshape(n, KH, D)
        v = plain.causal_conv_silu(pd[:, 2 * KH * D:C], w["v.conv"].double()).reshape(n, H, V)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        beta = torch.sigmoid(pd[:, C:])
        dec = torch.exp(-torch.exp(w["A_log"].double())[None, :, None]
                        * plain.softplus(ad + w["dt_bias"].double()).reshape(n, H, D))
        S = torch.zeros(H, D, V, dtype=torch.float64)
        o = torch.zeros(n, H, V, dtype=torch.float64)
        for t in range(n):
            for h in range(H):
                kt, qt = k[t, h // 2], q[t, h // 2]
                S[h] = dec[t, h][:, None] * S[h]
                S[h] = S[h] + kt[:, None] * (beta[t, h] * (v[t, h] - S[h].T @ kt))[None, :]
                o[t, h] = S[h].T @ qt
        want.append(o)
    dev = "cuda"
    state = torch.full((4, H * D * V + C * (taps - 1)), float("nan"), device=dev)
    for s in slots:
        state[s].zero_()
    conv_w = torch.cat([w["q.conv"], w["k.conv"], w["v.conv"]]).contiguous().to(dev)
    at = [0, 0, 0]
    got = [[], [], []]
    sizes = [3, 1, 7, 2, 1, 5, 2, 6]
    k = 0
    while any(a < n for a, n in zip(at, lens)):
        live = [r for r in (2, 0, 1) if at[r] < lens[r]]             # batch order differs from slot order
        take = []
        for r in live:
            m = min(sizes[k % len(sizes)], lens[r] - at[r])
            k += 1
            take.append(m)
        T = sum(take)
        p = torch.cat([p_all[r][at[r]:at[r] + m] for r, m in zip(live, take)]).to(dev)
        a = torch.cat([a_all[r][at[r]:at[r] + m] for r, m in zip(live, take)]).to(dev)
        cu = torch.tensor(np.concatenate([[0], np.cumsum(take)]), dtype=torch.int32, device=dev)
        rot = torch.tensor(sum(([i] * m for i, m in enumerate(take)), []), dtype=torch.int32, device=dev)
        sl = torch.tensor([slots[r] for r in live], dtype=torch.int32, device=dev)
        qn, kn, dec = (torch.empty(T * H * D, device=dev) for _ in range(3))
        vc, beta, o = torch.empty(T * H * V, device=dev), torch.empty(T * H, device=dev), torch.empty(T * H * V, device=dev)
        ops.delta_prepare(p, 0, C, a, conv_w, w["A_log"].to(dev), w["dt_bias"].to(dev), state, H * D * V, rot, cu, sl,
                          qn, kn, vc, beta, dec, H, KH, D, V, taps, D ** -0.5)
        ops.conv_state_update(p, 0, C, state, H * D * V, cu, sl, taps)
        ops.delta_recurrence(qn, kn, vc, beta, dec, state, cu, sl, o, H, D, V)
        o = o.view(T, H, V).cpu()
        t0 = 0
        for r, m in zip(live, take):
            got[r].append(o[t0:t0 + m])
            t0 += m
            at[r] += m
    for r in range(3):
        err = (torch.cat(got[r]).double() - want[r]).abs().max()
        assert err < 2e-5, (r, float(err))
    assert torch.isnan(state[1]).all()          # a slot nobody holds is not touched


def test_sublayer_kernels():
    from tiny_llm_amd.kernels import ops
    g = torch.Generator().manual_seed(3)
    T, H, F = 37, 72, 40
    y, x = torch.randn(T, H, generator=g) * 3, torch.randn(T, H, generator=g)
    wz, ls = torch.randn(H, generator=g) * 0.1, torch.rand(H, generator=g) + 0.5
    want = x.double() + plain.norm_around_zero(y.double(), wz.double(), 1e-5) * ls.double()
    xs = x.clone().cuda()
    copy = torch.empty(T, H, dtype=torch.bfloat16, device="cuda")
    ops.norm_scale_add(y.cuda(), (1.0 + wz).cuda(), 1e-5, xs, ls.cuda(), copy)
    assert (xs.cpu().double() - want).abs().max() < 1e-5
    assert torch.equal(copy.cpu(), xs.cpu().to(torch.bfloat16))
    gu = torch.randn(T, 2 * F, generator=g) * 3
    lim = 1.7
    gg, uu = torch.clamp(gu[:, :F].double(), max=lim), torch.clamp(gu[:, F:].double(), -lim, lim)
    z = torch.empty(T, F, device="cuda")
    ops.clamped_glu(gu.cuda(), z, lim, 1.702, 1.0)
    assert (z.cpu().double() - gg * torch.sigmoid(1.702 * gg) * (uu + 1)).abs().max() < 1e-5
    lg = (torch.randn(5, 33, generator=g) * 40).cuda()
    want = 25.0 * torch.tanh(lg.cpu().double() / 25.0)
    assert (ops.softcap(lg, 25.0).cpu().double() - want).abs().max() < 1e-4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_head_products(dtype):
    """The per-head products of steps with few rows, on views into wider rows, against an einsum."""
    from tiny_llm_amd.kernels import ops
    g = torch.Generator().manual_seed(2)
    for T, H, K, N, extra in ((1, 3, 24, 40, 8), (5, 2, 40, 16, 0), (11, 4, 128, 72, 16), (8, 1, 520, 33, 0)):
        x = torch.randn(T, H, K + extra, generator=g).to(dtype).cuda()
        w = (torch.randn(H, K, N, generator=g) / K ** 0.5).to(dtype).cuda()
        want = torch.einsum("thk,hkn->thn", x[:, :, :K].double().cpu(), w.double().cpu())
        for out_dtype in {dtype, torch.float32}:
            out = torch.full((T, H, N + extra), float("nan"), dtype=out_dtype, device="cuda")
            ops.head_products(x[:, :, :K], ops.head_product_weights(w), out[:, :, :N])
            tol = 1e-5 if out_dtype == torch.float32 else 2e-2
            assert (out[:, :, :N].double().cpu() - want).abs().max() < tol
            assert extra == 0 or torch.isnan(out[:, :, N:]).all()      # nothing is written beside the view


def test_head_gemm():
    """The same products for many rows on the matrix cores, with edges in every direction."""
    from tiny_llm_amd.kernels import ops
    g = torch.Generator().manual_seed(6)
    for T, H, K, N, extra in ((33, 3, 24, 40, 8), (200, 2, 40, 16, 0), (70, 4, 128, 72, 16), (64, 1, 520, 33, 8)):
        x = torch.randn(T, H, K + extra, generator=g).to(torch.bfloat16).cuda()
        w = (torch.randn(H, N, K, generator=g) / K ** 0.5).to(torch.bfloat16).cuda()
        want = torch.einsum("thk,hnk->thn", x[:, :, :K].double().cpu(), w.double().cpu())
        for out_dtype in (torch.bfloat16, torch.float32):
            out = torch.full((T, H, N + extra), float("nan"), dtype=out_dtype, device="cuda")
            ops.head_gemm(x[:, :, :K], w, out[:, :, :N])
            tol = 1e-4 if out_dtype == torch.float32 else 2e-2
            assert (out[:, :, :N].double().cpu() - want).abs().max() < tol
            assert extra == 0 or torch.isnan(out[:, :, N:]).all()


def test_command_line_and_seeded_sampling(tmp_path_factory):
    """bin/tiny_llm serves a Lufazen folder as it serves any other (config.json chooses the model);
    seeded sampling through the engine does not depend on what else is in the batch."""
    folder, cfg, w, reqs, ref, block = material("A", "float32", tmp_path_factory)
    prompt = reqs["r2"][:12]
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "tiny_llm"), "--model_path", folder,
                           "--nodo_sample", "--max_new_tokens=5", "--dtype", "float32", "--ignore_eos",
                           "--prompt_ids", ",".join(map(str, prompt))], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    got = [int(t) for t in proc.stdout.strip().splitlines()[-1].split()]
    seq = list(prompt)
    for _ in range(5):
        seq.append(int(plain.forward(cfg, w, seq)[-1].argmax()))
    assert got == seq[len(prompt):]
    from tiny_llm_amd import Engine, SamplingParams
    eng = Engine(folder, dtype="float32", kv_block_size=block, max_num_seqs=4, max_num_batched_tokens=64, max_model_len=256)
    params = SamplingParams(max_new_tokens=12, do_sample=True, temperature=0.9, top_k=40, top_p=0.95, seed=7,
                            ignore_eos=True)
    alone = eng.generate([prompt], params)[0]
    among = eng.generate([reqs["r0"][:30], prompt, reqs["r1"][:7]], params)[1]
    assert alone == among


def test_random_weights_from_a_configuration():
    """A configuration that names the two ranks itself runs with seeded random weights (no files), as
    the measurements do."""
    import copy
    from lufazen_util import MIX_A, RANKS_A
    from tiny_llm_amd import Engine, SamplingParams
    cfg = copy.deepcopy(MIX_A)
    for i, (ra, rg) in RANKS_A.items():
        cfg["layers"][i]["mixer"].update(decay_rank=ra, gate_rank=rg)
    eng = Engine(config=cfg, dtype="bfloat16", kv_block_size=16, max_num_seqs=2, max_num_batched_tokens=32,
                 max_model_len=128, weights_seed=3, init_std=0.05)
    out = eng.generate([random_tokens(20, cfg["vocab"], 1), random_tokens(3, cfg["vocab"], 2)],
                       SamplingParams.greedy(8, ignore_eos=True))
    assert [len(o) for o in out] == [8, 8] and all(0 <= t < cfg["vocab"] for o in out for t in o)


def test_latent_prefill_tiles_of_several_tokens():
    """The kernel of steps with many rows on tiles that hold several tokens: one request's 13 consecutive
    tokens in tiles of four (the last one of a single token), 20 heads (two tiles of heads, the second partly
    used), each head aiming at a key of its own; and 5 heads, where a wave holds three tokens."""
    from tiny_llm_amd.kernels import ops
    g = torch.Generator().manual_seed(8)
    n, kv_rank, rot, block = 420, 64, 16, 8
    lat = torch.randn(n, kv_rank, generator=g)
    lat = lat / lat.norm(dim=1, keepdim=True)
    rope = torch.randn(n, rot, generator=g) * 0.1
    table = torch.randperm(64, generator=g)[: -(-n // block)].tolist()
    pages_l, pages_r = _paged(lat, table, block, 64, torch.bfloat16), _paged(rope, table, block, 64, torch.bfloat16)
    bt = torch.tensor([table + [0] * (64 - len(table))], dtype=torch.int32, device="cuda")
    lat_r, rope_r = lat.to(torch.bfloat16).double(), rope.to(torch.bfloat16).double()
    for heads, first in ((20, 300), (5, 27)):
        T = 13
        per_tile = 4 * (16 // min(heads, 16))
        positions = torch.arange(first, first + T, dtype=torch.int32)
        qa = torch.randn(T, heads, kv_rank + rot, generator=g) * 0.3
        for t in range(T):
            for h in range(heads):
                qa[t, h, :kv_rank] += 50.0 * lat[(11 * h + 3 * t) % (first + t + 1)]
        starts = list(range(0, T, per_tile))
        tiles = (torch.zeros(len(starts), dtype=torch.int32, device="cuda"),
                 torch.tensor(starts, dtype=torch.int32, device="cuda"),
                 torch.tensor([min(per_tile, T - s0) for s0 in starts], dtype=torch.int32, device="cuda"))
        gate = torch.randn(T, heads, generator=g).to(torch.bfloat16)
        out = torch.empty(T, heads, kv_rank, dtype=torch.bfloat16, device="cuda")
        ops.latent_prefill(qa.cuda(), pages_l, pages_r, bt, tiles, positions.cuda(), out, 0.7, gate.cuda())
        for t in range(T):
            p = first + t
            for h in range(heads):
                s = (qa[t, h, :kv_rank].double() @ lat_r[:p + 1].T + qa[t, h, kv_rank:].double() @ rope_r[:p + 1].T) * 0.7
                want = torch.softmax(s, dim=0) @ lat_r[:p + 1] * torch.sigmoid(gate[t, h].double())
                assert (out[t, h].double().cpu() - want).abs().max() < 1e-2, (heads, t, h)
