"""The Vevapel architecture in the engine against the plain implementation of its equations
(tests/plain_vevapel.py): each mechanism alone, every way of cutting the work, pages and state slots
used again, captured steps, long decoding, generation through the entry point, and keys that a
crafted query singles out at the places where an index can be off by one."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_vevapel as plain
import traces
from vevapel_util import CONFIGS, MIX_A, as_double, make_folder, random_config, rounded, row_err, tame
from util import random_tokens

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# float32: everything is computed in 32 bits, what is left is the order of sums.  bfloat16: weights are
# rounded for the plain model too; the products' inputs and outputs are rounded in the engine only, the
# models are made tame so that this rounding is not amplified, and every token uses every expert (a logit
# that bfloat16 moves past its neighbour would otherwise choose another expert; the router's choices are
# compared in float32 and, with logits that are apart, at the part itself).  A fault of a mechanism (a key
# off by one, a chunk's edge, a lost state, a pass's vector left out) moves a row by its whole size in
# either precision.  The float32 figure: the plain model itself, run in float32, differs from its float64 run by
# up to 3.2e-4 of a row on the liveliest model here (twelve layer runs, scores sharpened three times; the engine, whose
# sums run in other orders, by up to 5.3e-4), by 8e-5 and less on the others.  The bfloat16 models are also tamed in
# their residual multiplier (`vevapel_util.tame`):
# rounding nothing but every sublayer's input to bfloat16 in the plain model (`round_inputs`, the one rounding no
# bfloat16 engine can avoid) then moves a row by 1.7e-2 at worst, where the untamed model moves by 1.2e-1.
TOL = {"float32": 1e-3, "bfloat16": 1e-1}
LENGTHS = {"A": [70, 133, 33, 200, 97, 64], "B": [1, 9, 40, 100, 150, 57], "odd": [31, 2, 77, 50],
           "loop_all": [30, 3, 66], "loop_one": [45, 8, 90, 2], "wide": [50, 7, 101], "attention": [40, 75, 130, 9], "diff": [40, 75, 130, 9],
           "delta": [24, 121, 48, 5], "moe": [24, 121, 48, 5]}

_cache = {}


def config_for(name, dtype):
    cfg, block = CONFIGS[name]
    return (tame(cfg) if dtype == "bfloat16" else cfg), block


def material(name, dtype, tmp_path_factory):
    key = (name, dtype)
    if key not in _cache:
        cfg, block = config_for(name, dtype)
        folder, w = make_folder(tmp_path_factory.mktemp(f"vevapel_{name}_{dtype}"), cfg, seed=11,
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
        st.fill_(12345)
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


CASES = [(n, "float32") for n in ("attention", "diff", "delta", "moe", "loop_all", "loop_one", "wide", "A", "B", "odd")] + \
        [(n, "bfloat16") for n in ("attention", "diff", "delta", "moe", "loop_one", "wide", "A", "B")]


@pytest.mark.parametrize("name,dtype", CASES)
def test_whole_tail_portions(name, dtype, tmp_path_factory):
    """Each request alone: whole, its tail token by token (chunks' edges pass under decoded tokens), and in
    portions down to two tokens (one-layer models of each sublayer, the loops, then the mixed models)."""
    folder, cfg, w, reqs, ref, block = material(name, dtype, tmp_path_factory)
    biggest = max(r64(len(t)) for t in reqs.values())
    for build in (traces.whole, traces.tail_one_by_one, traces.portions):
        steps = build(reqs)
        runner = make_runner(folder, dtype, block, biggest, max_seqs=1)
        worst = check(replay(runner, steps), steps, ref, TOL[dtype])
        print(f"{name} {dtype} {build.__name__}: worst {worst:.2e}")
        assert all_free(runner)


def test_odd_sizes_in_a_bfloat16_engine(tmp_path_factory):
    """A checkpoint stored in bfloat16 whose sizes are multiples of nothing, asked for in bfloat16: the float32
    kernels serve it (with a warning), mixed batches and portions agree with the plain model to float32's limit."""
    cfg, block = CONFIGS["odd"]
    folder, w = make_folder(tmp_path_factory.mktemp("vevapel_odd_bf16"), cfg, seed=4, store=torch.bfloat16)
    reqs = {f"r{i}": random_tokens(n, cfg["vocab"], 50 + i) for i, n in enumerate(LENGTHS["odd"])}
    ref = {rid: plain.forward(cfg, rounded(w), toks) for rid, toks in reqs.items()}
    steps, peak = traces.mixed(reqs, seed=3)
    with pytest.warns(RuntimeWarning, match="served in float32"):
        runner = make_runner(folder, "bfloat16", block, max(peak, max(r64(len(t)) for t in reqs.values())))
    assert runner.decoder.dtype == torch.float32
    for st in (steps, traces.portions(reqs)):
        check(replay(runner, st), st, ref, TOL["float32"])
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
    """Sizes nobody chose: width, head counts and sizes with and without a matrix-core kernel, keys wider and
    narrower than values, chunks from one position to more than the prompt and none, rotated dims, temperatures,
    taps, loops over any run of layers, layers without feed-forward, pages of 4 to 32 tokens; mixed batches,
    portions and whole prompts in both precisions."""
    import random
    drawn = random_config(seed)
    rng = random.Random(1000 + seed)
    block = rng.choice([4, 8, 16, 32])
    for dtype in ("float32", "bfloat16"):
        cfg = tame(drawn) if dtype == "bfloat16" else drawn
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
def test_layer_sizes_of_a_larger_model(dtype, tmp_path):
    """Three layers with heads of the sizes a model of some billions of weights has (heads of 128 and 64, four and
    two query heads a key head, a chunk that a prompt of 300 tokens crosses, experts of 64 hidden units), run twice:
    a whole prompt (the kernels for many rows), the same in portions, and a tail decoded token by token beside a
    second request."""
    from vevapel_util import attention, attention_2, delta, layer, model, moe
    big = model(256, 1031, [
        layer(attention(16, 4, 128, 128, (0.3, 50), 128 ** -0.5), moe(16, 4, 64)),
        layer(delta(8, 4, 128, 128, 4), moe(12, 3, 32)),
        layer(attention_2(8, 4, 64, 128, 180, 32, 0.2, 500000.0, 64 ** -0.5), moe(8, 2, 64)),
    ], loop=(0, 3, 2), scale=8.0)
    cfg = tame(big) if dtype == "bfloat16" else big
    folder, w = make_folder(tmp_path, cfg, seed=5, store=torch.bfloat16 if dtype == "bfloat16" else torch.float32,
                            sharpen=1.0 if dtype == "bfloat16" else 3.0)
    w64 = rounded(w) if dtype == "bfloat16" else as_double(w)
    reqs = {"long": random_tokens(300, cfg["vocab"], 1), "short": random_tokens(45, cfg["vocab"], 2)}
    ref = {rid: plain.forward(cfg, w64, toks) for rid, toks in reqs.items()}
    runner = make_runner(folder, dtype, 16, 384 + 64)
    for st in (traces.whole(reqs), traces.portions(reqs), traces.mixed(reqs, seed=1)[0]):
        worst = check(replay(runner, st), st, ref, TOL[dtype])
        assert all_free(runner)
        print(f"larger sizes {dtype}: worst {worst:.2e}")


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
    """One to four tokens: the convolutions reach back into zeros, the state starts empty, a softmax holds one key."""
    for name in ("A", "B"):
        folder, cfg, w, reqs, ref, block = material(name, "float32", tmp_path_factory)
        runner = make_runner(folder, "float32", block, 64)
        from tiny_llm_amd.engine.step import StepEntry
        for n in (1, 2, 3, 4):
            logits = runner.step([StepEntry("x", reqs["r3"][:n], list(range(n)))]).cpu()
            runner.finish("x")
            for i in range(n):
                assert row_err(logits[i], ref["r3"][i]) < TOL["float32"]


def test_long_decoding(tmp_path_factory):
    """Several hundred single-token steps: the states and the convolutions' inputs are carried from step to step
    in every pass of the loop, every page edge and every chunk's edge is crossed by decoded tokens, the query
    temperature steps up twenty times."""
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
    folder, cfg, w, reqs, ref, block = material("A", "float32", tmp_path_factory)
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


def test_preempted_requests_are_computed_again(tmp_path_factory):
    """A pool so small that requests are preempted and recomputed from their first token: their state slots start
    empty again in every pass and the tokens are the same."""
    folder, cfg, w, reqs, ref, block = material("A", "float32", tmp_path_factory)
    from tiny_llm_amd import Engine, SamplingParams
    prompts = [reqs["r0"][:60], reqs["r1"][:50], reqs["r3"][:40]]
    big = Engine(folder, dtype="float32", kv_block_size=block, max_num_seqs=3, max_num_batched_tokens=64, max_model_len=256)
    want = big.generate(prompts, SamplingParams.greedy(30, ignore_eos=True))
    small = Engine(folder, dtype="float32", kv_block_size=block, max_num_seqs=3, max_num_batched_tokens=64,
                   max_model_len=256, num_kv_blocks=11)
    assert small.generate(prompts, SamplingParams.greedy(30, ignore_eos=True)) == want
    small.runner.cache.audit()


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
    """bin/tiny_llm serves a Vevapel folder as it serves any other (config.json chooses the model);
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
    """A configuration written by hand runs with seeded random weights (no files), as the measurements do."""
    from tiny_llm_amd import Engine, SamplingParams
    eng = Engine(config=MIX_A, dtype="bfloat16", kv_block_size=16, max_num_seqs=2, max_num_batched_tokens=32,
                 max_model_len=128, weights_seed=3, init_std=0.05)
    out = eng.generate([random_tokens(20, MIX_A["vocab"], 1), random_tokens(3, MIX_A["vocab"], 2)],
                       SamplingParams.greedy(8, ignore_eos=True))
    assert [len(o) for o in out] == [8, 8] and all(0 <= t < MIX_A["vocab"] for o in out for t in o)


# ------------------------------------------------------------------ mechanisms alone
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
@pytest.mark.parametrize("chunk", [40, 1, 17, 64, 150, 0])
def test_chunked_mask_finds_one_key(kernel, chunk):
    """One query per place of interest is aligned with one key (and scaled so that this score stands out): the result
    must be that key's value.  Keys at the chunk's first place, at both sides of page edges, the query's own position,
    the first positions; the key just OUTSIDE the chunk (the last of the chunk before) and the one behind the query
    are louder still, and the mask must hide them.  Every attention kernel takes the chunk as a negative window.
    Chunk 0 is no chunk at all (the mixer without a mask): the one key then lies hundreds of positions back."""
    from tiny_llm_amd.kernels import ops
    dtype = torch.float32 if "float32" in kernel else torch.bfloat16
    g = torch.Generator().manual_seed(5)
    n, d, block, heads, kvh = 700, 32, 16, 6, 2
    keys = torch.randn(n, kvh, d, generator=g)
    keys = keys / keys.norm(dim=-1, keepdim=True)
    vals = torch.randn(n, kvh, d, generator=g)
    table = torch.randperm(64, generator=g)[: -(-n // block)].tolist()
    k_pages, v_pages = _paged_kv(keys, table, block, 64, dtype), _paged_kv(vals, table, block, 64, dtype)
    first = lambda pos: pos // chunk * chunk if chunk else 0
    places = {699, 650, 640, 639, 600, 599, 400, 399, 200, 199, 64, 63, 48, 47, 31, 16, 15, 1, 0,
              first(699), first(699) - 1, first(300), first(300) + chunk - 1, 300}
    cases = sorted({(pos, key) for pos in places if 0 <= pos < n
                    for key in (first(pos), pos, (first(pos) + pos) // 2, min(first(pos) + 1, pos))})
    T = len(cases)
    q = torch.zeros(T, heads, d)
    for i, (pos, key) in enumerate(cases):
        lo = first(pos)
        for h in range(heads):
            # head 0 aims at the case's key, the others at keys of their own inside the chunk
            target = key if h == 0 else lo + (key - lo + 3 * h) % (pos - lo + 1)
            q[i, h] = 30.0 * keys[target, h // (heads // kvh)]
            if pos + 1 < n:                       # the key behind the query would win if it were seen
                q[i, h] += 50.0 * keys[pos + 1, h // (heads // kvh)]
            if lo - 1 >= 0:                       # and so would the last key of the chunk before
                q[i, h] += 50.0 * keys[lo - 1, h // (heads // kvh)]
    positions = [c[0] for c in cases]
    pos_dev = torch.tensor(positions, dtype=torch.int32, device="cuda")
    bt = torch.tensor([table + [0] * (64 - len(table))], dtype=torch.int32, device="cuda")
    out = torch.empty(T, heads * d, dtype=dtype, device="cuda")
    qd = q.reshape(T, heads * d).to(dtype).cuda()
    each = torch.arange(T, dtype=torch.int32, device="cuda")
    tables = bt.repeat(T, 1).contiguous()         # every query a request of its own over the same pages
    window = -chunk
    if kernel.startswith("general"):
        ops.paged_attention(qd, k_pages, v_pages, bt, torch.zeros(T, dtype=torch.int32, device="cuda"), pos_dev, out,
                            heads, kvh, d, 1.0, window)
    elif "float32" in kernel and "many rows" in kernel:
        reps = -(-1024 // (T * kvh)) + 1
        big = torch.empty(T * reps, heads * d, dtype=dtype, device="cuda")
        n_t = T * reps
        tiles = (torch.arange(n_t, dtype=torch.int32, device="cuda"),) * 2 + (torch.ones(n_t, dtype=torch.int32, device="cuda"),)
        ops.attention_f32(qd.repeat(reps, 1), k_pages, v_pages, bt.repeat(n_t, 1).contiguous(), tiles, pos_dev.repeat(reps),
                          big, heads, kvh, d, 1.0, window)
        assert all(torch.equal(big[:T], big[r * T:(r + 1) * T]) for r in range(1, reps))
        out = big[:T]
    elif "float32" in kernel:
        chunks = -(-700 // ops.F32_CHUNK_KEYS) if "chunks" in kernel else 1
        part = torch.empty(chunks * T * heads * (d + 2), device="cuda") if chunks > 1 else None
        ops.attention_f32(qd, k_pages, v_pages, tables, None, pos_dev, out, heads, kvh, d, 1.0, window, chunks, part)
    elif "prompt" in kernel:
        splits = 3 if "split" in kernel else 1
        part = torch.empty(splits * T * heads * (d + 2), device="cuda") if splits > 1 else None
        ops.flash_prefill(qd, k_pages, v_pages, tables, (each, each.clone(), torch.ones_like(each)), pos_dev, out, heads, kvh,
                          d, 1.0, window, 4, splits, part)
    else:
        splits = 3 if "split" in kernel else 1
        part = torch.empty(splits * T * heads * (d + 2), device="cuda") if splits > 1 else None
        ops.flash_attention(qd, k_pages, v_pages, tables, None, pos_dev, out, heads, kvh, d, 1.0, window, splits, part)
    kr, vr, qr = keys.to(dtype).double(), vals.to(dtype).double(), q.to(dtype).double()
    out = out.double().cpu().reshape(T, heads, d)
    for i, pos in enumerate(positions):
        lo = first(pos)
        for h in range(heads):
            kv = h // (heads // kvh)
            p = torch.softmax(kr[lo:pos + 1, kv] @ qr[i, h], dim=-1)
            want = p @ vr[lo:pos + 1, kv]
            assert torch.isfinite(out[i, h]).all()
            assert (out[i, h] - want).abs().max() < (2e-5 if dtype == torch.float32 else 2e-2), (pos, h)


@pytest.mark.parametrize("kernel", ["general float32", "matrix cores float32", "matrix cores bfloat16, prompt"])
@pytest.mark.parametrize("chunk", [24, 100])
def test_chunked_attention_of_a_prompts_portion(kernel, chunk):
    """A portion of a prompt behind cached tokens, cut in the middle of a chunk and of a page: tiles that hold
    several tokens whose chunks differ."""
    from tiny_llm_amd.kernels import ops
    dtype = torch.float32 if "float32" in kernel else torch.bfloat16
    g = torch.Generator().manual_seed(8)
    n, d, block, heads, kvh, start = 190, 32, 16, 4, 2, 57
    keys, vals = torch.randn(n, kvh, d, generator=g) * 1.5, torch.randn(n, kvh, d, generator=g)
    q = torch.randn(n - start, heads, d, generator=g) * 1.5
    table = torch.randperm(16, generator=g)[: -(-n // block)].tolist()
    k_pages, v_pages = _paged_kv(keys, table, block, 16, dtype), _paged_kv(vals, table, block, 16, dtype)
    T = n - start
    pos_dev = torch.arange(start, n, dtype=torch.int32, device="cuda")
    bt = torch.tensor([table + [0] * (16 - len(table))], dtype=torch.int32, device="cuda")
    out = torch.empty(T, heads * d, dtype=dtype, device="cuda")
    qd = q.reshape(T, heads * d).to(dtype).cuda()
    width = 16 // (heads // kvh)
    if kernel.startswith("general"):
        ops.paged_attention(qd, k_pages, v_pages, bt, torch.zeros(T, dtype=torch.int32, device="cuda"), pos_dev, out,
                            heads, kvh, d, d ** -0.5, -chunk)
    else:
        if "prompt" in kernel:
            width *= 4
        tok0 = torch.arange(0, T, width, dtype=torch.int32, device="cuda")
        tiles = (torch.zeros_like(tok0), tok0, torch.clamp(T - tok0, max=width).to(torch.int32))
        if "prompt" in kernel:
            ops.flash_prefill(qd, k_pages, v_pages, bt, tiles, pos_dev, out, heads, kvh, d, d ** -0.5, -chunk, 4, 1, None)
        else:
            ops.attention_f32(qd, k_pages, v_pages, bt, tiles, pos_dev, out, heads, kvh, d, d ** -0.5, -chunk)
    kr, vr, qr = keys.to(dtype).double(), vals.to(dtype).double(), q.to(dtype).double()
    pos = torch.arange(n)
    allowed = plain.same_chunk(pos, chunk)[start:]
    s = torch.einsum("ihd,jhd->hij", qr, kr.repeat_interleave(heads // kvh, 1)) * d ** -0.5
    s = s.masked_fill(~allowed[None], float("-inf"))
    want = torch.einsum("hij,jhv->ihv", torch.softmax(s, -1), vr.repeat_interleave(heads // kvh, 1))
    got = out.double().cpu().reshape(T, heads, d)
    assert (got - want).abs().max() < (2e-5 if dtype == torch.float32 else 3e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("maps,dim,vdim,rot,pairing,norm", [(1, 24, 16, 0, "half", "whole"), (2, 16, 24, 8, "half", None),
                                                            (2, 6, 11, 4, "interleaved", "unit"), (1, 40, 8, 40, "half", "whole"),
                                                            (1, 8, 8, 0, "half", None)])
def test_attn_prepare(dtype, maps, dim, vdim, rot, pairing, norm):
    """Bias, the norm over a token's whole query (key) projection with its weights, rotation of part of every map of
    every head, the unit norm, the query temperature; queries out map by map in rows of D with zeros behind dim, keys
    of each map and values into pages at scattered slots with zeros behind their sizes; a negative slot stores nothing."""
    from tiny_llm_amd.kernels import ops
    from tiny_llm_amd.parts.rotary import angle_tables
    g = torch.Generator().manual_seed(3)
    T, H, G, block, eps, coef, every = 11, 4, 2, 4, 1e-5, 0.7, 5
    D = -(-max(dim, vdim) // 16) * 16
    qc, kc, vc = H * maps * dim, G * maps * dim, G * vdim
    p = torch.randn(T, qc + kc + vc + 5, generator=g)
    bias = torch.randn(qc + kc + vc, generator=g)
    norm_w = 1.0 + 0.3 * torch.randn(qc + kc, generator=g)
    positions = torch.randint(0, 500, (T,), generator=g)
    positions[0] = 0
    slots = torch.randperm(40, generator=g)[:T].to(torch.int32)
    slots[4] = -1
    cos = sin = None
    if rot:
        cos, sin = angle_tables(rot, 777.0, 512, "cuda")
    pages = [torch.full((10, G, block, D), float("nan"), dtype=dtype, device="cuda") for _ in range(maps + 1)]
    q = torch.full((maps, T, H * D), float("nan"), dtype=dtype, device="cuda")
    ops.attn_prepare(p.cuda(), bias.cuda(), norm_w.cuda() if norm == "whole" else None, positions.to(torch.int32).cuda(),
                     cos, sin, slots.cuda(), q, pages[:maps], pages[maps], H, G, maps, dim, vdim, qc + kc, rot, pairing,
                     norm == "whole", norm == "unit", eps, (coef, every))
    a = p[:, :qc + kc + vc].double() + bias.double()
    qa, ka, va = a[:, :qc], a[:, qc:qc + kc], a[:, qc + kc:].reshape(T, G, vdim)
    if norm == "whole":
        qa = plain.unit_rms(qa, eps) * norm_w[:qc].double()
        ka = plain.unit_rms(ka, eps) * norm_w[qc:].double()
    qa, ka = qa.reshape(T, H, maps, dim), ka.reshape(T, G, maps, dim)
    if rot:
        if pairing == "half":
            qa, ka = plain.rotate_half(qa, positions, rot, 777.0), plain.rotate_half(ka, positions, rot, 777.0)
        else:
            def pairs(x):
                f = 777.0 ** (-2.0 * torch.arange(rot // 2, dtype=torch.float64) / rot)
                ang = positions.double()[:, None] * f[None, :]
                c, s = torch.cos(ang)[:, None, None, :], torch.sin(ang)[:, None, None, :]
                y = x.clone()
                u, v = x[..., 0:rot:2], x[..., 1:rot:2]
                y[..., 0:rot:2], y[..., 1:rot:2] = u * c - v * s, v * c + u * s
                return y
            qa, ka = pairs(qa), pairs(ka)
    if norm == "unit":
        qa, ka = plain.unit_rms(qa, eps), plain.unit_rms(ka, eps)
    qa = qa * plain.query_temperature(positions, coef, every)[:, None, None, None]
    rel = 1e-5 if dtype == torch.float32 else 2.0 ** -8         # a bfloat16 result is its value rounded once
    close = lambda got, want: bool(((got - want).abs() <= rel * (want.abs() + 1.0)).all())
    got_q = q.double().cpu().reshape(maps, T, H, D)
    for m in range(maps):
        assert close(got_q[m][..., :dim], qa[:, :, m])
        assert (got_q[m][..., dim:] == 0).all()
    for t in range(T):
        s = int(slots[t])
        if s < 0:
            continue
        for m in range(maps):
            row = pages[m][s // block, :, s % block].double().cpu()
            assert close(row[:, :dim], ka[t, :, m]) and (row[:, dim:] == 0).all()
        row = pages[maps][s // block, :, s % block].double().cpu()
        assert close(row[:, :vdim], va[t]) and (row[:, vdim:] == 0).all()
    used = {int(s) for s in slots if s >= 0}
    for s in range(40):
        if s not in used:
            assert all(torch.isnan(pg[s // block, :, s % block]).all() for pg in pages)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("two,sub_norm,gate,tail", [(True, True, "element", 0), (False, False, "head", 8), (False, False, None, 0),
                                                    (True, False, "head", 8)])
def test_attn_finish(dtype, two, sub_norm, gate, tail):
    """Behind the attention kernel: the maps' difference, the norm per head, the constant, the gates, the values'
    columns picked out of rows of D, and the column of ones for an output bias."""
    from tiny_llm_amd.kernels import ops
    g = torch.Generator().manual_seed(4)
    T, H, vdim, D, lam, eps, scale = 9, 5, 24, 32, 0.37, 1e-5, 0.7
    a0 = torch.randn(T, H * D, generator=g).to(dtype if tail else torch.float32)    # float32 in, either type out
    a1 = torch.randn(T, H * D, generator=g).to(a0.dtype)
    gates = torch.randn(T, H if gate == "head" else H * vdim, generator=g)
    z = torch.full((T, H * vdim + tail), float("nan"), dtype=dtype, device="cuda")
    ops.attn_finish(a0.cuda(), a1.cuda() if two else None, gates.cuda() if gate else None, z, H, vdim, lam, sub_norm, eps,
                    scale, gate, tail)
    o = a0.double().reshape(T, H, D)[..., :vdim]
    if two:
        o = o - lam * a1.double().reshape(T, H, D)[..., :vdim]
    if sub_norm:
        o = plain.unit_rms(o, eps)
    o = o * scale
    if gate == "head":
        o = o * torch.sigmoid(gates.double())[:, :, None]
    elif gate == "element":
        o = o * torch.sigmoid(gates.double()).reshape(T, H, vdim)
    got = z.double().cpu()
    assert (got[:, :H * vdim] - o.reshape(T, H * vdim)).abs().max() < (1e-5 if dtype == torch.float32 else 4e-2)
    if tail:
        assert torch.equal(got[:, H * vdim:], torch.tensor([1.0] + [0.0] * (tail - 1), dtype=torch.float64).repeat(T, 1))


def test_sandwich_norm_kernel():
    """x <- x + m LN(y) and, in the same kernel, the next norm of the new x; rows of odd and of large width."""
    from tiny_llm_amd.kernels import ops
    g = torch.Generator().manual_seed(6)
    for W in (50, 192, 2048, 5000):
        x, y = torch.randn(7, W, generator=g) * 3 + 1, torch.randn(7, W, generator=g) * 0.5 - 2
        w1, b1, w2, b2 = (torch.randn(W, generator=g) for _ in range(4))
        want_x = x.double() + 0.7 * plain.layer_norm(y.double(), w1.double(), b1.double(), 1e-5)
        want_h = plain.layer_norm(want_x, w2.double(), b2.double(), 3e-6)
        for dtype in (torch.float32, torch.bfloat16):
            xd = x.clone().cuda()
            h = torch.empty(7, W, dtype=dtype, device="cuda")
            ops.layer_norm_add(y.cuda(), w1.cuda(), b1.cuda(), xd, 0.7, 1e-5, then=(w2.cuda(), b2.cuda(), 3e-6, h))
            assert (xd.double().cpu() - want_x).abs().max() < 1e-4
            assert (h.double().cpu() - want_h).abs().max() < (1e-4 if dtype == torch.float32 else 5e-2)
        xd = x.clone().cuda()
        ops.layer_norm_add(y.cuda(), w1.cuda(), b1.cuda(), xd, 0.7, 1e-5)
        assert (xd.double().cpu() - want_x).abs().max() < 1e-4


def test_stream_join_and_loop_entry():
    """[x | x0] as one operand, the pass's vector as the rows the product adds to: x <- W_in [x ; x0] + step."""
    from tiny_llm_amd.kernels import ops
    g = torch.Generator().manual_seed(7)
    T, W = 13, 40
    x, x0, vec, w_in = (torch.randn(s, generator=g) for s in ((T, W), (T, W), (W,), (W, 2 * W)))
    want = torch.cat([x, x0], -1).double() @ w_in.double().T + vec.double()
    for dtype, tol in ((torch.float32, 1e-4), (torch.bfloat16, 1e-1)):
        operand = torch.empty(T, 2 * W, dtype=dtype, device="cuda")
        out = torch.full((T, W), float("nan"), device="cuda")
        ops.stream_join(x.cuda(), x0.cuda(), vec.cuda(), operand, out)
        assert torch.equal(out.cpu(), vec.repeat(T, 1)) and torch.equal(operand.cpu(), torch.cat([x, x0], -1).to(dtype))
        ops.linear(operand, w_in.to(dtype).cuda(), out, out)
        assert (out.double().cpu() - want).abs().max() < tol


@pytest.mark.parametrize("experts,top", [(6, 2), (8, 3), (64, 6), (5, 5), (130, 4), (1, 1), (16, 2)])
def test_router_kernel_with_a_bias(experts, top):
    """The router kernel with a bias per expert and one group: the largest logits, largest first, weighed by the
    softmax over the chosen logits alone (also when the other logits are far larger in size than the chosen ones'
    differences, and when a chosen logit lies far below the best)."""
    from tiny_llm_amd.kernels import ops
    g = torch.Generator().manual_seed(experts * 7 + top)
    T = 37
    z = torch.randn(T, experts, generator=g) * 3.0
    z[0] += 80.0                                   # large logits: only differences count
    if experts > 1:
        z[1, 0] += 60.0                            # one expert far above the rest
    bias = torch.randn(experts, generator=g)
    ids = torch.empty(T, top, dtype=torch.int32, device="cuda")
    wts = torch.empty(T, top, device="cuda")
    ops.moe_route(z.cuda(), ids, wts, 1, 1, 1.0, bias.cuda())
    val, want_ids = torch.topk((z + bias).double(), top, dim=-1)
    assert torch.equal(ids.cpu().long(), want_ids)
    assert (wts.double().cpu() - torch.softmax(val, -1)).abs().max() < 1e-6


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("tokens", [5, 40, 700])
def test_gated_experts_by_every_route(dtype, tokens):
    """The routed feed-forward part alone with gated experts and a router bias, by each of its three routes (rows
    against their own expert, tiles of one expert's rows, runs of rows through the tiled product), with an expert that
    no token chooses and logits that are apart, so that both precisions choose alike."""
    from tiny_llm_amd.parts.moe import RoutedMoE
    g = torch.Generator().manual_seed(tokens)
    W, E, top, F = 64, 5, 2, 24
    tdt = torch.float32 if dtype == "float32" else torch.bfloat16
    names = {}
    for e in range(E):
        names[f"m.e{e}.gate"], names[f"m.e{e}.up"] = torch.randn(F, W, generator=g) / 8, torch.randn(F, W, generator=g) / 8
        names[f"m.e{e}.down"] = torch.randn(W, F, generator=g) / 5
    # the router reads the first channels: channel e of h is expert e's logit, so the choice is plain to see
    router = torch.zeros(E, W)
    router[:, :E] = torch.eye(E) * 4.0
    names["m.router"], names["m.router.b"] = router, torch.tensor([0.0, 0.5, -100.0, 0.25, 0.0])     # expert 2 is never chosen
    h = torch.randn(tokens, W, generator=g) * 0.5
    h[:, :E] = torch.stack([torch.randperm(E, generator=g).float() for _ in range(tokens)])           # logits 4 apart
    w = {k: v.to(tdt) for k, v in names.items()}
    part = RoutedMoE("m", tdt, torch.device("cuda"), hidden_size=W, num_experts=E, top=top, intermediate_size=F,
                     activation="swiglu", router_bias=True)
    part.bind({k: v.cuda() for k, v in w.items()})
    out = part.forward(h.to(tdt).cuda(), None, None)
    wd = {k[2:]: v.double() for k, v in w.items()}
    want = plain.moe(h.to(tdt).double(), wd, {"router": {"top": top}})
    ids, _ = plain.route(h.to(tdt).double(), wd["router"], wd["router.b"], top)
    assert 2 not in ids
    err = (out.double().cpu() - want).abs().max() / want.abs().max()
    assert err < (1e-5 if dtype == "float32" else 3e-2)


@pytest.mark.parametrize("H,G,D,V,taps", [(4, 2, 16, 8, 4), (3, 3, 24, 40, 2), (2, 1, 64, 64, 3), (1, 1, 128, 128, 4),
                                          (3, 1, 5, 9, 3)])
def test_delta_state_over_slots_and_tiny_portions(H, G, D, V, taps):
    """The delta rule's kernels alone with one decay per head, full-rank pre-activations and the SiLU gate: three
    requests of unequal length in slots out of order, fed in portions of 1 to 7 tokens (single tokens take the one-kernel
    decode step), against the plain scan over each whole sequence."""
    from tiny_llm_amd.parts.delta_rule import ChannelDelta

    class Ctx:
        pass

    g = torch.Generator().manual_seed(9)
    W, eps = 40, 1e-5
    part = ChannelDelta("m", torch.float32, torch.device("cuda"), hidden_size=W, num_heads=H, num_kv_heads=G, head_dim=D,
                        value_dim=V, conv_taps=taps, decay_rank=0, gate_rank=0, eps=eps, decay="head", gate="silu")
    w = {}
    for s in part.weights():
        t = torch.randn(*s.shape, generator=g)
        w[s.name] = t * (2.0 / W ** 0.5 if len(s.shape) == 2 and s.shape[-1] == W else 0.5)
    w["m.norm"] = 1.0 + 0.2 * torch.randn(V, generator=g)
    part.bind({k: v.cuda() for k, v in w.items()})
    lens, slots = [23, 9, 40], [2, 0, 3]
    hs = [torch.randn(n, W, generator=g) for n in lens]
    wd = {k[2:]: v.double() for k, v in w.items()}
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "conv": taps}
    want = [plain.delta(h.double(), wd, m, eps) for h in hs]
    state = torch.full((4, part.state_spec().shape[0]), float("nan"), device="cuda")
    for s in slots:
        state[s].zero_()
    at, got = [0, 0, 0], [[], [], []]
    sizes = [3, 1, 7, 2, 1, 5, 2, 6, 1, 1, 1, 1, 1, 1]
    k = 0
    while any(a < n for a, n in zip(at, lens)):
        live = [r for r in (2, 0, 1) if at[r] < lens[r]]             # batch order differs from slot order
        take = []
        for r in live:
            take.append(min(sizes[k % len(sizes)], lens[r] - at[r]))
            k += 1
        if k % 5 == 0:
            take = [1] * len(live)                                    # a step of single tokens: the decode kernel
        h = torch.cat([hs[r][at[r]:at[r] + n] for r, n in zip(live, take)]).cuda()
        ctx = Ctx()
        ctx.cu_seqlens_q = torch.tensor([0] + list(np.cumsum(take)), dtype=torch.int32, device="cuda")
        ctx.req_of_token = torch.tensor([i for i, n in enumerate(take) for _ in range(n)], dtype=torch.int32, device="cuda")
        ctx.state_slots = torch.tensor([slots[r] for r in live], dtype=torch.int32, device="cuda")
        ctx.max_q_len, ctx.num_requests = max(take), len(live)
        out = part.forward(h, ctx, None, state, None).cpu()
        o = 0
        for r, n in zip(live, take):
            got[r].append(out[o:o + n].clone())
            o += n
            at[r] += n
    for r in range(3):
        err = (torch.cat(got[r]).double() - want[r]).abs().max() / want[r].abs().max()
        assert err < 2e-4, (r, float(err))
    assert torch.isnan(state[1]).all()
