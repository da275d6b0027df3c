"""The Fofapel architecture in the engine against the plain implementation of its equations
(tests/plain_fofapel.py): each mechanism alone, every way of cutting the work, pages and state slots
used again, captured steps, long decoding, generation through the entry point, and keys that a
crafted query singles out at the places where an index can be off by one."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_fofapel as plain
import traces
from fofapel_util import CONFIGS, as_double, make_folder, rounded, row_err
from util import random_tokens

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# float32: everything is computed in 32 bits, what is left is the order of sums.  bfloat16: weights are
# rounded for the plain model too; the products' inputs and outputs are rounded in the engine only, and
# the models are made tame so that this rounding is not amplified.  A fault of a mechanism (a key off by
# one, a state lost, a wrong slot) moves a row by its whole size in either precision.
TOL = {"float32": 2e-4, "bfloat16": 1e-1}
LENGTHS = {"A": [70, 133, 33, 200, 97, 64], "B": [1, 9, 40, 100, 150, 57], "dense": [40, 75, 130, 9],
           "moe": [24, 121, 48, 5]}

_cache = {}


def material(name, dtype, tmp_path_factory):
    key = (name, dtype)
    if key not in _cache:
        cfg, block = CONFIGS[name]
        folder, w = make_folder(tmp_path_factory.mktemp(f"fofapel_{name}_{dtype}"), cfg, seed=11,
                                store=torch.bfloat16 if dtype == "bfloat16" else torch.float32,
                                sharpen=1.0 if dtype == "bfloat16" else 3.0)
        w64 = rounded(w) if dtype == "bfloat16" else as_double(w)
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
@pytest.mark.parametrize("name", ["dense", "moe", "A", "B"])
def test_whole_tail_portions(name, dtype, tmp_path_factory):
    """Each request alone: whole, its tail token by token (the windows pass over decoded tokens), and in
    portions down to two tokens (one-layer models of each feed-forward, then the two mixed models)."""
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


@pytest.mark.parametrize("seed", range(10))
def test_configurations_drawn_at_random(seed, tmp_path):
    """Sizes nobody chose: width, heads and head sizes (with and without a matrix-core attention kernel), windows
    from one token to more than the prompt, rotated dims, time-mix shapes, ranks, feed-forwards of every kind and
    none, pages of 4 to 32 tokens; mixed batches and portions in both precisions against the plain model."""
    import random
    from fofapel_util import random_config
    cfg = random_config(seed)
    rng = random.Random(1000 + seed)
    block = rng.choice([4, 8, 16, 32])
    for dtype in ("float32", "bfloat16"):
        folder, w = make_folder(tmp_path / dtype, cfg, seed=seed, store=torch.bfloat16 if dtype == "bfloat16" else torch.float32,
                                sharpen=1.0 if dtype == "bfloat16" else 3.0)
        w64 = rounded(w) if dtype == "bfloat16" else as_double(w)
        reqs = {f"r{i}": random_tokens(n, cfg["vocab"], 7 * seed + i) for i, n in enumerate([rng.randrange(1, 140) for _ in range(5)])}
        ref = {rid: plain.forward(cfg, w64, toks) for rid, toks in reqs.items()}
        steps, peak = traces.mixed(reqs, seed=seed)
        runner = make_runner(folder, dtype, block, max(peak, max(r64(len(t)) for t in reqs.values())))
        for st in (steps, traces.portions(reqs), traces.whole(reqs)):
            worst = check(replay(runner, st), st, ref, TOL[dtype])
            assert all_free(runner)
        print(f"seed {seed} {dtype}: worst {worst:.2e}")


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
    """One to four tokens: the shifted input of the first token is zero, its state is empty, and its
    softmax holds one key and the sink."""
    folder, cfg, w, reqs, ref, block = material("B", "float32", tmp_path_factory)
    runner = make_runner(folder, "float32", block, 64)
    from tiny_llm_amd.engine.step import StepEntry
    for n in (1, 2, 3, 4):
        logits = runner.step([StepEntry("x", reqs["r3"][:n], list(range(n)))]).cpu()
        runner.finish("x")
        for i in range(n):
            assert row_err(logits[i], ref["r3"][i]) < TOL["float32"]


def test_long_decoding(tmp_path_factory):
    """Several hundred single-token steps: the recurrent state is carried that far, every page edge is
    crossed, every window passes over decoded tokens, pages behind the windows are given back."""
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


def test_command_line_and_seeded_sampling(tmp_path_factory):
    """bin/tiny_llm serves a Fofapel folder as it serves any other (config.json chooses the model);
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
    """A configuration written by hand (it names the decay's rank itself) runs with seeded random weights
    (no files), as the measurements do; the experts' table then holds distinct experts in every row."""
    from fofapel_util import MIX_A
    from tiny_llm_amd import Engine, SamplingParams
    eng = Engine(config=MIX_A, dtype="bfloat16", kv_block_size=16, max_num_seqs=2, max_num_batched_tokens=32,
                 max_model_len=128, weights_seed=3, init_std=0.05)
    out = eng.generate([random_tokens(20, MIX_A["vocab"], 1), random_tokens(3, MIX_A["vocab"], 2)],
                       SamplingParams.greedy(8, ignore_eos=True))
    assert [len(o) for o in out] == [8, 8] and all(0 <= t < MIX_A["vocab"] for o in out for t in o)
    table = eng.runner.decoder.layers[0].by_role["ffn"].table.cpu()
    assert table.shape == (MIX_A["vocab"], 3) and int(table.min()) >= 0 and int(table.max()) < 5
    assert all(len(set(row.tolist())) == 3 for row in table)


# ------------------------------------------------------------------ kernels with crafted inputs
def _paged_kv(rows: torch.Tensor, table, block, n_blocks, dtype):
    """rows [n, kv_heads, d] laid into pages [n_blocks, kv_heads, block, d] at the blocks `table` names; NaN elsewhere."""
    n, g, d = rows.shape
    pages = torch.full((n_blocks, g, block, d), float("nan"), dtype=dtype, device="cuda")
    for j in range(n):
        pages[table[j // block], :, j % block] = rows[j].to(dtype)
    return pages


ATTENTION_KERNELS = ["general float32", "general bfloat16", "matrix cores float32", "matrix cores float32, chunks",
                     "matrix cores float32, many rows", "matrix cores bfloat16", "matrix cores bfloat16, split keys",
                     "matrix cores bfloat16, prompt", "matrix cores bfloat16, prompt, split keys"]


@pytest.mark.parametrize("kernel", ATTENTION_KERNELS)
@pytest.mark.parametrize("window", [40, 1, 17])
def test_window_and_sink_find_one_key(kernel, window):
    """One query per place of interest is aligned with one key (and scaled so that this score stands out):
    the result must be that key's value times what the sink leaves.  Keys at the window's first place, at
    both sides of page edges, the query's own position, the first positions; the key just OUTSIDE the
    window and the one behind the query are louder still, and the mask must hide them.  One query is
    turned away from every key it sees: the sink then takes nearly all of the weight."""
    from tiny_llm_amd.kernels import ops
    dtype = torch.float32 if "float32" in kernel else torch.bfloat16
    g = torch.Generator().manual_seed(5)
    n, d, block, heads, kvh = 700, 32, 16, 6, 2
    keys = torch.randn(n, kvh, d, generator=g)
    keys = keys / keys.norm(dim=-1, keepdim=True)
    vals = torch.randn(n, kvh, d, generator=g)
    table = torch.randperm(64, generator=g)[: -(-n // block)].tolist()
    k_pages, v_pages = _paged_kv(keys, table, block, 64, dtype), _paged_kv(vals, table, block, 64, dtype)
    back = [0, 1, window - 1, window // 2]
    cases = [(pos, max(pos - b, 0)) for pos in (699, 650, 64, 63, 48, 47, 31, 16, 15, 1, 0) for b in back]
    cases = sorted(set(cases))
    T = len(cases) + 1
    q = torch.zeros(T, heads, d)
    for i, (pos, key) in enumerate(cases):
        for h in range(heads):
            # head 0 aims at the case's key, the others at keys of their own inside the window
            lo = max(pos - window + 1, 0)
            target = key if h == 0 else lo + (key - lo + 3 * h) % (pos - lo + 1)
            q[i, h] = 30.0 * keys[target, h // (heads // kvh)]
            if pos + 1 < n:                       # the key behind the query would win if it were seen
                q[i, h] += 50.0 * keys[pos + 1, h // (heads // kvh)]
            if pos - window >= 0:                 # and so would the one the window has just left
                q[i, h] += 50.0 * keys[pos - window, h // (heads // kvh)]
    for h in range(heads):                        # the last query: a score of -15 with every key it sees
        seen = keys[300 - window + 1:301, h // (heads // kvh)].double()
        q[T - 1, h] = (torch.linalg.pinv(seen) @ torch.full((seen.shape[0],), -15.0, dtype=torch.float64)).float()
    positions = [c[0] for c in cases] + [300]
    pos_dev = torch.tensor(positions, dtype=torch.int32, device="cuda")
    bt = torch.tensor([table + [0] * (64 - len(table))], dtype=torch.int32, device="cuda")
    out = torch.empty(T, heads * d, dtype=dtype, device="cuda")
    qd = q.reshape(T, heads * d).to(dtype).cuda()
    each = torch.arange(T, dtype=torch.int32, device="cuda")
    tables = bt.repeat(T, 1).contiguous()         # every query a request of its own over the same pages
    if kernel.startswith("general"):
        ops.paged_attention(qd, k_pages, v_pages, bt, torch.zeros(T, dtype=torch.int32, device="cuda"), pos_dev, out,
                            heads, kvh, d, 1.0, window, sink=True)
    elif "float32" in kernel and "many rows" in kernel:
        # a thousand query tiles and more: the kernel that gives a wave a tile
        reps = -(-1024 // (T * kvh)) + 1
        big = torch.empty(T * reps, heads * d, dtype=dtype, device="cuda")
        n_t = T * reps
        tiles = (torch.arange(n_t, dtype=torch.int32, device="cuda"),) * 2 + (torch.ones(n_t, dtype=torch.int32, device="cuda"),)
        ops.attention_f32(qd.repeat(reps, 1), k_pages, v_pages, bt.repeat(n_t, 1).contiguous(), tiles, pos_dev.repeat(reps),
                          big, heads, kvh, d, 1.0, window, sink=True)
        assert all(torch.equal(big[:T], big[r * T:(r + 1) * T]) for r in range(1, reps))
        out = big[:T]
    elif "float32" in kernel:
        chunks = -(-700 // ops.F32_CHUNK_KEYS) if "chunks" in kernel else 1
        part = torch.empty(chunks * T * heads * (d + 2), device="cuda") if chunks > 1 else None
        ops.attention_f32(qd, k_pages, v_pages, tables, None, pos_dev, out, heads, kvh, d, 1.0, window, chunks, part,
                          sink=True)
    elif "prompt" in kernel:
        splits = 3 if "split" in kernel else 1
        part = torch.empty(splits * T * heads * (d + 2), device="cuda") if splits > 1 else None
        ops.flash_prefill(qd, k_pages, v_pages, tables, (each, each.clone(), torch.ones_like(each)), pos_dev, out, heads, kvh,
                          d, 1.0, window, 4, splits, part, sink=True)
    else:
        splits = 3 if "split" in kernel else 1
        part = torch.empty(splits * T * heads * (d + 2), device="cuda") if splits > 1 else None
        ops.flash_attention(qd, k_pages, v_pages, tables, None, pos_dev, out, heads, kvh, d, 1.0, window, splits, part,
                            sink=True)
    kr, vr, qr = keys.to(dtype).double(), vals.to(dtype).double(), q.to(dtype).double()
    out = out.double().cpu().reshape(T, heads, d)
    for i, pos in enumerate(positions):
        lo = max(pos - window + 1, 0)
        for h in range(heads):
            kv = h // (heads // kvh)
            s = kr[lo:pos + 1, kv] @ qr[i, h]
            p = plain.sink_softmax(s[None, :], torch.ones(1, s.numel(), dtype=torch.bool))[0]
            want = p @ vr[lo:pos + 1, kv]
            assert torch.isfinite(out[i, h]).all()
            assert (out[i, h] - want).abs().max() < (2e-5 if dtype == torch.float32 else 2e-2), (pos, h)
    if window <= d:                               # (more keys than dims: no query is away from all of them)
        assert out[T - 1].abs().max() < 1e-3      # the sink took the weight


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("pairing,rot", [("interleaved", 8), ("interleaved", 24), ("half", 12), ("interleaved", 0)])
def test_qk_prepare(dtype, pairing, rot):
    """Bias, rotation of part of a head in either pairing, unit root mean square, queries out, keys and the
    unrotated keys (as values) into pages at scattered slots; a negative slot stores nothing."""
    from tiny_llm_amd.kernels import ops
    from tiny_llm_amd.parts.rotary import angle_tables
    g = torch.Generator().manual_seed(3)
    T, H, G, D, block, eps = 11, 3, 1, 24, 4, 1e-5
    p = torch.randn(T, (H + G) * D + 8, generator=g)
    bias = torch.randn((H + G) * D, generator=g)
    positions = torch.randint(0, 500, (T,), generator=g)
    slots = torch.randperm(40, generator=g)[:T].to(torch.int32)
    slots[4] = -1
    cos = sin = None
    if rot:
        cos, sin = angle_tables(rot, 777.0, 512, "cuda")
    k_pages = torch.full((10, G, block, D), float("nan"), dtype=dtype, device="cuda")
    v_pages = torch.full_like(k_pages, float("nan"))
    q = torch.empty(T, H * D, dtype=dtype, device="cuda")
    ops.qk_prepare(p.cuda(), bias.cuda(), positions.to(torch.int32).cuda(), cos, sin, slots.cuda(), q, k_pages, v_pages,
                   H, G, D, rot, pairing, True, eps, True)
    a = (p[:, :(H + G) * D].double() + bias.double()).reshape(T, H + G, D)
    r = a.clone()
    if rot:
        if pairing == "interleaved":
            r = plain.rotate_pairs(a, positions, rot, 777.0)
        else:
            f = 777.0 ** (-2.0 * torch.arange(rot // 2, dtype=torch.float64) / rot)
            ang = positions.double()[:, None] * f[None, :]
            c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
            u, v = a[..., :rot // 2], a[..., rot // 2:rot]
            r = torch.cat([u * c - v * s, v * c + u * s, a[..., rot:]], dim=-1)
    r = plain.rms_unit(r, eps)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert (q.double().cpu().reshape(T, H, D) - r[:, :H]).abs().max() < tol
    for t in range(T):
        s = int(slots[t])
        if s < 0:
            continue
        assert (k_pages[s // block, :, s % block].double().cpu() - r[t, H:]).abs().max() < tol
        assert (v_pages[s // block, :, s % block].double().cpu() - a[t, H:]).abs().max() < tol * 4
    used = {int(s) for s in slots if s >= 0}
    for s in range(40):
        if s not in used:
            assert torch.isnan(k_pages[s // block, :, s % block]).all() and torch.isnan(v_pages[s // block, :, s % block]).all()


@pytest.mark.parametrize("H,D", [(3, 24), (1, 80), (2, 16), (4, 64), (1, 256)])
def test_time_mix_state_over_slots_and_tiny_portions(H, D):
    """The shift and the recurrence kernels alone: three requests of unequal length in slots out of order,
    fed in portions of 1 to 7 tokens, against the plain recurrence over each whole sequence; heads that are
    no power of two of the kernel's 4-channel slices, narrow, and as wide as it takes."""
    from tiny_llm_amd.kernels import ops
    g = torch.Generator().manual_seed(9)
    W, S = 40, H * D
    lens, slots = [23, 9, 40], [2, 0, 3]
    w0 = torch.rand(S, generator=g) * 3.0 - 3.0
    u = torch.randn(H, D, generator=g) * 0.5
    mu = torch.rand(2, W, generator=g)
    xs = [torch.randn(n, 4 * S, generator=g) * 0.5 for n in lens]        # r | k | v | decay pre-activation
    hs = [torch.randn(n, W, generator=g) for n in lens]
    want_o, want_mix = [], []
    for x, h in zip(xs, hs):
        n = x.shape[0]
        xd = x.double()
        r, k, v = (xd[:, i * S:(i + 1) * S].reshape(n, H, D) for i in range(3))
        dec = torch.exp(-torch.exp(xd[:, 3 * S:] + w0.double())).reshape(n, H, D)
        want_o.append(plain.time_mix_recurrence(r, k, v, dec, u.double()))
        want_mix.append(torch.stack([plain.shifted_mix(h.double(), m.double()) for m in mu]))
    dev = "cuda"
    s_floats = ops.time_mix_state_floats(H, D, D)
    state = torch.full((4, s_floats + W), float("nan"), device=dev)
    for s in slots:
        state[s].zero_()
    at, got_o, got_mix = [0, 0, 0], [[], [], []], [[], [], []]
    sizes = [3, 1, 7, 2, 1, 5, 2, 6, 1, 1, 1, 1, 1, 1]
    k = 0
    while any(a < n for a, n in zip(at, lens)):
        live = [r for r in (2, 0, 1) if at[r] < lens[r]]             # batch order differs from slot order
        take = []
        for r in live:
            take.append(min(sizes[k % len(sizes)], lens[r] - at[r]))
            k += 1
        x = torch.cat([xs[r][at[r]:at[r] + m] for r, m in zip(live, take)]).to(dev)
        h = torch.cat([hs[r][at[r]:at[r] + m] for r, m in zip(live, take)]).to(dev)
        T = x.shape[0]
        cu = torch.tensor([0] + list(np.cumsum(take)), dtype=torch.int32, device=dev)
        req = torch.tensor([i for i, m in enumerate(take) for _ in range(m)], dtype=torch.int32, device=dev)
        sl = torch.tensor([slots[r] for r in live], dtype=torch.int32, device=dev)
        mixes = torch.empty(2, T, W, device=dev)
        single = all(m == 1 for m in take)            # such a step's shift saves the tokens itself
        ops.shift_mix(h, state, s_floats, req, cu, sl, mu.to(dev), mixes, save_single=single)
        if not single:
            ops.shift_save(h, state, s_floats, cu, sl)
        o = torch.empty(T * S, device=dev)
        ops.time_mix_recurrence(x, 0, S, 2 * S, 3 * S, w0.to(dev), u.reshape(-1).to(dev), state, cu, sl, o, H, D, D)
        o = o.reshape(T, H, D).cpu()
        t = 0
        for r, m in zip(live, take):
            got_o[r].append(o[t:t + m])
            got_mix[r].append(mixes[:, t:t + m].cpu())
            at[r] += m
            t += m
    for r in range(3):
        o = torch.cat(got_o[r]).double()
        scale = want_o[r].abs().max()
        assert (o - want_o[r]).abs().max() < 2e-5 * max(1.0, float(scale)), (r, H, D)
        assert (torch.cat(got_mix[r], dim=1).double() - want_mix[r]).abs().max() < 1e-5
    assert torch.isnan(state[1]).all()                                # the slot nobody holds was never touched


def test_sum_norm_and_gated_units():
    """Layer norm behind the sum (with and without a sublayer's result, odd widths, a copy in bfloat16), on
    gathered rows, the gated GELU, the sigmoid gate per head, and the head norm with a weight per head and a
    SiLU gate."""
    from tiny_llm_amd.kernels import ops
    g = torch.Generator().manual_seed(1)
    for W in (40, 333, 2304):
        T = 7
        x, y = torch.randn(T, W, generator=g) * 3 + 1, torch.randn(T, W, generator=g)
        w, b = torch.randn(W, generator=g), torch.randn(W, generator=g)
        for yy in (y, None):
            want = plain.layer_norm(2.5 * x.double() + (yy.double() if yy is not None else 0.0), w.double(), b.double(), 1e-5)
            xd, copy = x.clone().cuda(), torch.empty(T, W, dtype=torch.bfloat16, device="cuda")
            ops.layer_norm_sum(yy.cuda() if yy is not None else None, w.cuda(), b.cuda(), xd, 2.5, 1e-5, copy)
            assert (xd.double().cpu() - want).abs().max() < 2e-5
            assert (copy.double().cpu() - want).abs().max() < 5e-2
        rows = torch.tensor([5, 0, 5, 2], dtype=torch.int32)
        out = torch.empty(4, W, device="cuda")
        ops.layer_norm_rows(x.cuda(), w.cuda(), b.cuda(), 1e-5, out, rows.cuda())
        want = plain.layer_norm(x.double()[rows.long()], w.double(), b.double(), 1e-5)
        assert (out.double().cpu() - want).abs().max() < 2e-5
    gu = torch.randn(5, 2 * 24, generator=g) * 2
    z = torch.empty(5, 24, device="cuda")
    ops.gelu_glu(gu.cuda(), z)
    assert (z.double().cpu() - plain.gelu_tanh(gu[:, :24].double()) * gu[:, 24:].double()).abs().max() < 1e-5
    a, gates = torch.randn(5, 3 * 8, generator=g), torch.randn(5, 16, generator=g)
    out = torch.empty(5, 24, device="cuda")
    ops.head_gate(a.cuda(), gates.cuda()[:, 4:7], out, 3, 8, 1.7)
    want = a.double().reshape(5, 3, 8) * torch.sigmoid(gates[:, 4:7].double())[:, :, None] * 1.7
    assert (out.double().cpu().reshape(5, 3, 8) - want).abs().max() < 1e-5
    o, wn, gt = torch.randn(5, 3 * 8, generator=g), torch.randn(24, generator=g), torch.randn(5, 24, generator=g)
    out = torch.empty(5, 24, device="cuda")
    ops.head_norm_gate(o.cuda().reshape(-1), wn.cuda(), gt.cuda(), out, 3, 8, 1e-5, "silu", 0.9)
    want = plain.rms_unit(o.double().reshape(5, 3, 8), 1e-5).reshape(5, 24) * wn.double() * \
        (gt.double() * torch.sigmoid(gt.double())) * 0.9
    assert (out.double().cpu() - want).abs().max() < 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_table_moe_kernels(dtype):
    """Rows against the weights of their own experts, looked up by token id; the sum of a token's experts on
    top of a base with a factor per row."""
    from tiny_llm_amd.kernels import ops
    g = torch.Generator().manual_seed(2)
    T, W, F, E, top, V = 9, 40, 24, 5, 3, 50
    h = torch.randn(T, W, generator=g).to(dtype)
    w_up = (torch.randn(E, 2 * F, W, generator=g) / W ** 0.5).to(dtype)
    w_dn = (torch.randn(E, W, F, generator=g) / F ** 0.5).to(dtype)
    table = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(V)]).to(torch.int32)
    tokens = torch.randint(0, V, (T,), generator=g).to(torch.int32)
    gu = torch.empty(T * top, 2 * F, dtype=dtype, device="cuda")
    ops.table_moe_up(h.cuda(), w_up.cuda(), tokens.cuda(), table.cuda(), gu)
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    for t in range(T):
        for j in range(top):
            want = w_up[table[tokens[t], j]].double() @ h[t].double()
            assert (gu[t * top + j].double().cpu() - want).abs().max() < tol
    z = torch.randn(T * top, F, generator=g).to(dtype)
    base, scale = torch.randn(T, W, generator=g), torch.rand(T, generator=g)
    out = base.clone().cuda()
    ops.table_moe_down(z.cuda(), w_dn.cuda(), tokens.cuda(), table.cuda(), out, 1.0 / top, out, scale.cuda())
    for t in range(T):
        want = base[t].double() * scale[t].double()
        for j in range(top):
            want = want + w_dn[table[tokens[t], j]].double() @ z[t * top + j].double() / top
        assert (out[t].double().cpu() - want).abs().max() < tol
    sg = torch.randn(W, generator=g).to(dtype)
    s = torch.empty(T, device="cuda")
    ops.row_dot_sigmoid(h.cuda(), sg.cuda(), s)
    assert (s.double().cpu() - torch.sigmoid(h.double() @ sg.double())).abs().max() < 1e-5


@pytest.mark.parametrize("T,top,E,N,K", [(70, 3, 5, 72, 40), (33, 1, 3, 300, 64), (200, 2, 2, 16, 104), (64, 2, 9, 260, 32)])
def test_rows_grouped_by_expert_on_the_matrix_cores(T, top, E, N, K):
    """Many rows: sorted by expert on the device, tiles of 32 rows of one expert; experts with no row, with one,
    with more than a tile; column counts that fill no tile; every row against its own expert's weights."""
    from tiny_llm_amd.kernels import ops
    g = torch.Generator().manual_seed(T)
    V = 40
    h = torch.randn(T, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(E, N, K, generator=g) / K ** 0.5).to(torch.bfloat16)
    table = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(V)]).to(torch.int32)
    if E > 2:
        table[table == E - 1] = 0 if top == 1 else table[table == E - 1]      # (top 1: the last expert gets no row)
    tokens = torch.randint(0, V, (T,), generator=g).to(torch.int32)
    rows = T * top
    plan = torch.full((ops.moe_plan_ints(rows, E),), -7, dtype=torch.int32, device="cuda")
    ops.moe_plan(tokens.cuda(), table.cuda(), plan, E)
    counts = plan[:E].cpu()
    want_counts = torch.bincount(table[tokens.long()].reshape(-1).long(), minlength=E)
    assert torch.equal(counts.long(), want_counts)
    mt = ops.moe_max_tiles(rows, E)
    sorted_rows = plan[3 * E + 2 + 3 * mt:3 * E + 2 + 3 * mt + rows].cpu()
    assert sorted(sorted_rows.tolist()) == list(range(rows))
    for out_dtype, a, div in ((torch.bfloat16, h, top), (torch.float32, h.repeat_interleave(top, 0), 1)):
        out = torch.full((rows, N), float("nan"), dtype=out_dtype, device="cuda")
        ops.grouped_rows_gemm(a.cuda(), div, w.cuda(), plan, out)
        for r in range(rows):
            want = w[table[tokens[r // top], r % top]].double() @ h[r // top].double()
            assert (out[r].double().cpu() - want).abs().max() < (3e-2 if out_dtype == torch.bfloat16 else 1e-4), (r, out_dtype)
    y, base, sc = torch.randn(rows, N, generator=g), torch.randn(T, N, generator=g), torch.rand(T, generator=g)
    out = base.clone().cuda()
    ops.moe_combine(y.cuda().reshape(-1), out, top, 0.5, out, sc.cuda())
    want = base.double() * sc.double()[:, None] + 0.5 * y.double().reshape(T, top, N).sum(1)
    assert (out.double().cpu() - want).abs().max() < 1e-5


@pytest.mark.parametrize("T,top,E,N,K", [(600, 2, 3, 72, 40), (300, 1, 4, 264, 64), (400, 3, 3, 512, 104)])
def test_runs_of_an_experts_rows_through_the_tiled_product(T, top, E, N, K):
    """Very many rows: every expert's rows copied side by side into runs of 256, the tiled product with a weight
    matrix per run (runs without rows skipped), and the sum of a token's rows looked up where they went."""
    from tiny_llm_amd.kernels import ops
    g = torch.Generator().manual_seed(T)
    V, R = 40, ops.MOE_RUN_ROWS
    h = torch.randn(T, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(E, N, K, generator=g) / K ** 0.5).to(torch.bfloat16)
    table = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(V)]).to(torch.int32)
    if top == 1:
        table[table == E - 1] = 0                 # an expert without rows
    tokens = torch.randint(0, V, (T,), generator=g).to(torch.int32)
    rows = T * top
    cap = ops.moe_max_tiles(rows, E, R) * R
    plan = torch.full((ops.moe_plan_ints(rows, E, R),), -7, dtype=torch.int32, device="cuda")
    ops.moe_plan(tokens.cuda(), table.cuda(), plan, E, R)
    runs = ops.moe_tile_experts(plan, rows, E, R)
    hp = torch.full((cap, K), float("nan"), dtype=torch.bfloat16, device="cuda")
    pos = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    ops.moe_gather(h.cuda(), top, plan, rows, E, R, hp, pos)
    where = pos.cpu().long()
    assert len(set(where.tolist())) == rows and int(where.min()) >= 0 and int(where.max()) < cap
    for out_dtype in (torch.bfloat16, torch.float32):
        out = torch.full((cap, N), float("nan"), dtype=out_dtype, device="cuda")
        ops.linear_grouped(hp, w.cuda(), runs, out)
        got = out.double().cpu()[where]
        for r in range(0, rows, 7):
            e = int(table[tokens[r // top], r % top])
            assert int(runs[where[r] // R]) == e
            want = w[e].double() @ h[r // top].double()
            assert (got[r] - want).abs().max() < (3e-2 if out_dtype == torch.bfloat16 else 1e-4), (r, out_dtype)
    y = torch.randn(cap, N, generator=g)
    base, sc = torch.randn(T, N, generator=g), torch.rand(T, generator=g)
    out = base.clone().cuda()
    ops.moe_combine_at(y.cuda(), pos, out, top, 0.5, out, sc.cuda())
    want = base.double() * sc.double()[:, None] + 0.5 * y.double()[where].reshape(T, top, N).sum(1)
    assert (out.double().cpu() - want).abs().max() < 1e-5
