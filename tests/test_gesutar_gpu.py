"""The Gesutar architecture in the engine against the plain implementation of its equations
(tests/plain_gesutar.py): each mechanism alone, every way of cutting the work, pages and state slots
used again, captured steps, long decoding, generation through the entry point, and keys that a
crafted query singles out at the places where an index can be off by one."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_gesutar as plain
import traces
from gesutar_util import CONFIGS, MIX_A, as_double, every_expert, make_folder, random_config, rounded, row_err
from util import random_tokens

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# float32: everything is computed in 32 bits, what is left is the order of sums.  bfloat16: weights are
# rounded for the plain model too; the products' inputs and outputs are rounded in the engine only, the
# models are made tame so that this rounding is not amplified, and every token uses every expert (a score
# that bfloat16 moves past its neighbour would otherwise choose another expert; the router's choices are
# compared in float32 and, with scores that are apart, at the part itself).  A fault of a mechanism (a key
# off by one, a sink left out, a wrong previous token) moves a row by its whole size in either precision.
TOL = {"float32": 2e-4, "bfloat16": 1e-1}
LENGTHS = {"A": [70, 133, 33, 200, 97, 64], "B": [1, 9, 40, 100, 150, 57], "odd": [31, 2, 77, 50],
           "attention": [40, 75, 130, 9], "moe": [24, 121, 48, 5], "no_pairs": [30, 3, 66]}

_cache = {}


def config_for(name, dtype):
    cfg, block = CONFIGS[name]
    return (every_expert(cfg) if dtype == "bfloat16" else cfg), block


def material(name, dtype, tmp_path_factory):
    key = (name, dtype)
    if key not in _cache:
        cfg, block = config_for(name, dtype)
        folder, w = make_folder(tmp_path_factory.mktemp(f"gesutar_{name}_{dtype}"), cfg, seed=11,
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


CASES = [(n, "float32") for n in ("attention", "moe", "A", "B", "odd", "no_pairs")] + \
        [(n, "bfloat16") for n in ("attention", "moe", "A", "B")]


@pytest.mark.parametrize("name,dtype", CASES)
def test_whole_tail_portions(name, dtype, tmp_path_factory):
    """Each request alone: whole, its tail token by token (the windows pass over decoded tokens), and in
    portions down to two tokens (one-layer models of each sublayer, then the mixed models)."""
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
    folder, w = make_folder(tmp_path_factory.mktemp("gesutar_odd_bf16"), cfg, seed=4, store=torch.bfloat16)
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
    """Sizes nobody chose: width, head counts and sizes, latents with and without a matrix-core kernel, windows
    from one token to more than the prompt and none, rotated dims, routers with and without groups, layers
    without feed-forward, pages of 4 to 32 tokens; mixed batches, portions and whole prompts in both precisions."""
    import random
    drawn = random_config(seed)
    rng = random.Random(1000 + seed)
    block = rng.choice([4, 8, 16, 32])
    for dtype in ("float32", "bfloat16"):
        cfg = every_expert(drawn) if dtype == "bfloat16" else drawn
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
    """Two layers with heads and latents of the sizes a model of some billions of weights has (sixteen heads of
    128 + 64 query/key dims, latents of 512 and 384, windows that a prompt of 300 tokens passes): a whole prompt (the
    kernels for many rows), the same in portions, and a tail decoded token by token beside a second request."""
    from gesutar_util import layer, mixer, model, moe
    big = model(256, 1031, [
        layer(mixer(16, 128, 64, 128, 512, 200, 64, 10000.0, 192 ** -0.5), moe(16, 4, 64, (4, 2), 1.0, 128)),
        layer(mixer(32, 64, 32, 64, 384, 90, 32, 500000.0, 96 ** -0.5), moe(12, 3, 32, (3, 2), 2.0, None)),
    ], bigram=(4093, 31, 17), scale=8.0)
    cfg = every_expert(big) if dtype == "bfloat16" else big
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
    """One to four tokens: the first takes the pair table's last row, its softmax holds one key and the sink."""
    folder, cfg, w, reqs, ref, block = material("B", "float32", tmp_path_factory)
    runner = make_runner(folder, "float32", block, 64)
    from tiny_llm_amd.engine.step import StepEntry
    for n in (1, 2, 3, 4):
        logits = runner.step([StepEntry("x", reqs["r3"][:n], list(range(n)))]).cpu()
        runner.finish("x")
        for i in range(n):
            assert row_err(logits[i], ref["r3"][i]) < TOL["float32"]


def test_long_decoding(tmp_path_factory):
    """Several hundred single-token steps: the previous token is carried from step to step, every page edge is
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
    held = [sum(b >= 0 for b in runner.cache.block_table("long", g)) for g in range(len(runner.cache.groups))]
    assert held[1] <= 2 and held[2] == -(-330 // block)        # the window of seven, the one longer than the prompt


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


def test_preempted_requests_are_computed_again(tmp_path_factory):
    """A pool so small that requests are preempted and recomputed from their first token: the previous token's
    slot starts empty again and the tokens are the same."""
    folder, cfg, w, reqs, ref, block = material("B", "float32", tmp_path_factory)
    from tiny_llm_amd import Engine, SamplingParams
    prompts = [reqs["r4"][:60], reqs["r3"][:50], reqs["r5"][:40]]
    big = Engine(folder, dtype="float32", kv_block_size=block, max_num_seqs=3, max_num_batched_tokens=64, max_model_len=256)
    want = big.generate(prompts, SamplingParams.greedy(30, ignore_eos=True))
    small = Engine(folder, dtype="float32", kv_block_size=block, max_num_seqs=3, max_num_batched_tokens=64,
                   max_model_len=256, num_kv_blocks=22)
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
    """bin/tiny_llm serves a Gesutar folder as it serves any other (config.json chooses the model);
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
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_pair_embedding_over_slots_and_portions(dtype):
    """Three requests in state slots out of order, fed in portions of one to five tokens, a slot handed to a new
    request in between: every row is the token's row times the scale plus the pair row of (token before, token)."""
    from tiny_llm_amd.kernels import ops
    g = torch.Generator().manual_seed(1)
    V, H, buckets, mp, mc, scale = 50, 24, 13, 1000003, 77, 2.5
    table = torch.randn(V, H, generator=g).to(dtype)
    pairs = torch.randn(buckets + 1, H, generator=g).to(dtype)
    state = torch.full((4, 1), 999, dtype=torch.int32, device="cuda")
    seqs = {s: random_tokens(n, V, s) for s, n in ((3, 17), (0, 9), (2, 12))}
    done = {s: 0 for s in seqs}
    w = {"embed": table.double(), "bigram": pairs.double()}
    conf = {"scale": scale, "bigram": {"buckets": buckets, "mul_prev": mp, "mul_cur": mc}}
    want = {s: plain.embed(t, w, conf) for s, t in seqs.items()}
    sizes = [1, 3, 2, 5, 1, 1, 4]
    k = 0
    while any(done[s] < len(seqs[s]) for s in seqs):
        toks, pos, req, cu, slots, rows = [], [], [], [0], [], []
        for s in seqs:
            n = min(sizes[k % len(sizes)], len(seqs[s]) - done[s])
            k += 1
            if n == 0:
                continue
            if done[s] == 0:
                state[s] = 0                     # what admission does
            toks += seqs[s][done[s]:done[s] + n]
            pos += range(done[s], done[s] + n)
            req += [len(slots)] * n
            rows += [(s, p) for p in range(done[s], done[s] + n)]
            slots.append(s)
            cu.append(len(toks))
            done[s] += n
        dev = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")
        out = torch.empty(len(toks), H, dtype=torch.float32, device="cuda")
        ops.embedding_pairs(dev(toks), dev(pos), dev(req), dev(cu), dev(slots), state, table.cuda(), pairs.cuda(), out,
                            mp, mc, scale)
        for i, (s, p) in enumerate(rows):
            assert (out[i].double().cpu() - want[s][p]).abs().max() < 1e-5, (s, p)
        for s in seqs:
            if done[s]:
                assert int(state[s]) == seqs[s][done[s] - 1]
    assert int(state[1]) == 999                  # a slot nobody held


@pytest.mark.parametrize("experts,top,groups,keep", [(6, 2, 3, 2), (8, 3, 1, 1), (64, 6, 8, 3), (5, 5, 1, 1), (130, 4, 10, 2),
                                                     (9, 3, 3, 1), (1, 1, 1, 1)])
def test_router_kernel(experts, top, groups, keep):
    from tiny_llm_amd.kernels import ops
    g = torch.Generator().manual_seed(experts)
    T = 200
    z = (3.0 * torch.randn(T, experts + 3, generator=g))[:, :experts]          # rows wider apart than they are long
    ids = torch.empty(T, top, dtype=torch.int32, device="cuda")
    wts = torch.empty(T, top, dtype=torch.float32, device="cuda")
    ops.moe_route(z.cuda(), ids, wts, groups, keep, 1.7)
    r = {"experts": experts, "top": top, "scale": 1.7}
    if groups > 1:
        r["groups"] = {"count": groups, "keep": keep}
    ref_ids, ref_w = plain.route(z.double(), r)
    order = ref_ids.argsort(dim=1)
    got_order = ids.cpu().long().argsort(dim=1)
    assert torch.equal(ids.cpu().long().gather(1, got_order), ref_ids.gather(1, order))
    assert (wts.cpu().double().gather(1, got_order) - ref_w.gather(1, order)).abs().max() < 1e-6
    assert (wts.cpu()[:, :-1] >= wts.cpu()[:, 1:]).all()                         # largest first


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("tokens", [5, 40, 700])
def test_routed_experts_by_every_route(dtype, tokens):
    """The routed feed-forward alone at few rows (each against its own expert), many (tiles of one expert's rows)
    and very many (runs of rows per expert), with tokens whose scores are apart so that both sides choose alike;
    one expert's router row is made so that it receives no token."""
    from tiny_llm_amd.parts.moe import RoutedMoE
    tdt = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    W, E, top, F, Fs = 64, 8, 3, 24, 40
    m = {"router": {"experts": E, "top": top, "scale": 1.5, "groups": {"count": 4, "keep": 3}}, "shared": {"ff": Fs}}
    g = torch.Generator().manual_seed(tokens)
    w = {f"e{e}.up": torch.randn(F, W, generator=g) / 8 for e in range(E)}
    w.update({f"e{e}.down": torch.randn(W, F, generator=g) / 5 for e in range(E)})
    w["router"] = torch.randn(E, W, generator=g) / 2
    w["router"][5] = 0.0
    w["router"][5, 0] = -5.0                     # every token's first element is large: expert 5 is chosen by nobody
    w["shared.up"], w["shared.down"] = torch.randn(Fs, W, generator=g) / 8, torch.randn(W, Fs, generator=g) / 6
    w = {k: v.to(tdt) for k, v in w.items()}
    w64 = {k: v.double() for k, v in w.items()}
    h = torch.randn(4 * tokens, W, generator=g)
    h[:, 0] += 4.0
    h = h.to(tdt)
    z = h.double() @ w64["router"].T
    chosen = plain.route(z, m["router"])[0].sort(dim=1).values
    apart = torch.ones(z.shape[0], dtype=torch.bool)
    for _ in range(6):                           # tokens whose choice survives a change of the logits by a few per cent
        moved = z * (1.0 + 0.03 * torch.randn(z.shape, generator=g, dtype=torch.float64))
        apart &= (plain.route(moved, m["router"])[0].sort(dim=1).values == chosen).all(dim=1)
    h = h[apart][:tokens]
    assert h.shape[0] == tokens and not (chosen[apart][:tokens] == 5).any()
    part = RoutedMoE("mlp", tdt, torch.device("cuda"), hidden_size=W, num_experts=E, top=top, intermediate_size=F,
                     groups=4, keep=3, scale=1.5, shared={"intermediate_size": Fs})
    part.bind({"mlp." + k: v.cuda() for k, v in w.items()})
    got = part.forward(h.cuda().contiguous(), None, None).double().cpu()
    want = plain.moe(h.double(), w64, m)
    err = (got - want).abs().max() / want.abs().max()
    print(f"{dtype} {tokens} tokens: {err:.2e}")
    assert err < (1e-5 if dtype == "float32" else 2e-2)


def _latent_pages(rows, table, block, n_blocks, dtype):
    n, d = rows.shape
    pages = torch.full((n_blocks, block, d), float("nan"), dtype=dtype, device="cuda")
    for j in range(n):
        pages[table[j // block], j % block] = rows[j].to(dtype)
    return pages


LATENT_KERNELS = ["general float32", "general bfloat16", "matrix cores", "matrix cores, split keys", "matrix cores, many rows"]


@pytest.mark.parametrize("kernel", LATENT_KERNELS)
@pytest.mark.parametrize("window,heads", [(40, 6), (1, 20), (17, 3), (0, 4)])
def test_latent_window_and_sink_find_one_key(kernel, window, heads):
    """One query per place of interest is aligned with one cached latent (and scaled so that this score stands
    out): the result must be that latent times what the sink leaves.  Keys at the window's first place, at both
    sides of page edges, the query's own position, the first positions, hundreds back without a window; the key
    just OUTSIDE the window and the one behind the query are louder still, and the mask must hide them.  Every
    head has a sink of its own, one of them far above every score: that head's result is nearly nothing."""
    from tiny_llm_amd.kernels import ops
    dtype = torch.float32 if "float32" in kernel else torch.bfloat16
    g = torch.Generator().manual_seed(5)
    n, C, R, block = 700, 32, 8, 16
    lat = torch.randn(n, C, generator=g)
    lat = lat / lat.norm(dim=-1, keepdim=True)
    kr = 0.3 * torch.randn(n, R, generator=g)
    rows = torch.cat([lat, kr], dim=1)
    table = torch.randperm(64, generator=g)[: -(-n // block)].tolist()
    l_pages, r_pages = _latent_pages(lat, table, block, 64, dtype), _latent_pages(kr, table, block, 64, dtype)
    sinks = torch.randn(heads, generator=g)
    sinks[heads - 1] = 200.0
    span = window if window else 700
    back = [0, 1, span - 1, span // 2]
    cases = sorted({(pos, max(pos - b, 0)) for pos in (699, 650, 64, 63, 48, 47, 31, 16, 15, 1, 0) for b in back})
    T = len(cases)
    q = torch.zeros(T, heads, C + R)
    for i, (pos, key) in enumerate(cases):
        lo = max(pos - span + 1, 0)
        for h in range(heads):
            target = key if h == 0 else lo + (key - lo + 3 * h) % (pos - lo + 1)
            q[i, h] = 30.0 * rows[target]
            if pos + 1 < n:                       # the key behind the query would win if it were seen
                q[i, h] += 50.0 * rows[pos + 1]
            if window and pos - window >= 0:      # and so would the one the window has just left
                q[i, h] += 50.0 * rows[pos - window]
    positions = [c[0] for c in cases]
    pos_dev = torch.tensor(positions, dtype=torch.int32, device="cuda")
    bt = torch.tensor([table + [0] * (64 - len(table))], dtype=torch.int32, device="cuda")
    tables = bt.repeat(T, 1).contiguous()         # every query a request of its own over the same pages
    each = torch.arange(T, dtype=torch.int32, device="cuda")
    out = torch.empty(T, heads, C, dtype=dtype, device="cuda")
    qd, sk = q.cuda(), sinks.cuda()
    if kernel.startswith("general"):
        ops.latent_attention(qd, l_pages, r_pages, bt, torch.zeros(T, dtype=torch.int32, device="cuda"), pos_dev, out, 1.0,
                             None, window, sk)
    elif "many rows" in kernel:
        ops.latent_prefill(qd, l_pages, r_pages, tables, (each, each.clone(), torch.ones_like(each)), pos_dev, out, 1.0,
                           None, window, sk)
    else:
        splits = 3 if "split" in kernel else 1
        part = torch.empty(splits * T * heads * (C + 2), device="cuda") if splits > 1 else None
        ops.latent_flash(qd, l_pages, r_pages, tables, None, pos_dev, out, 1.0, None, splits, part, window, sk)
    rr, lr = torch.cat([lat.to(dtype), kr.to(dtype)], dim=1).double(), lat.to(dtype).double()
    out = out.double().cpu()
    for i, pos in enumerate(positions):
        lo = max(pos - span + 1, 0)
        for h in range(heads):
            s = rr[lo:pos + 1] @ q[i, h].double()
            p = plain.sink_softmax(s[None, :], torch.ones(1, s.numel(), dtype=torch.bool), sinks[h].double())[0]
            want = p @ lr[lo:pos + 1]
            assert torch.isfinite(out[i, h]).all()
            assert (out[i, h] - want).abs().max() < (2e-5 if dtype == torch.float32 else 2e-2), (pos, h)
    assert out[:, heads - 1].abs().max() < 1e-2         # the sink far above every score took the weight


@pytest.mark.parametrize("kernel", ["general float32", "matrix cores", "matrix cores, many rows"])
@pytest.mark.parametrize("window,heads", [(9, 6), (40, 3), (0, 16)])
def test_latent_attention_of_a_prompt(kernel, window, heads):
    """One request's portion of 150 tokens behind 37 cached ones: tiles hold several tokens of the request, and
    every row sees its own window."""
    from tiny_llm_amd.kernels import ops
    from tiny_llm_amd.engine.step import tile_lists
    dtype = torch.float32 if "float32" in kernel else torch.bfloat16
    g = torch.Generator().manual_seed(window + heads)
    n0, T, C, R, block = 37, 150, 48, 16, 8
    n = n0 + T
    lat, kr = torch.randn(n, C, generator=g), torch.randn(n, R, generator=g)
    table = torch.randperm(40, generator=g)[: -(-n // block)].tolist()
    l_pages, r_pages = _latent_pages(lat, table, block, 40, dtype), _latent_pages(kr, table, block, 40, dtype)
    q = torch.randn(T, heads, C + R, generator=g)
    sinks = torch.randn(heads, generator=g)
    pos_dev = torch.arange(n0, n, dtype=torch.int32, device="cuda")
    bt = torch.tensor([table + [0] * (40 - len(table))], dtype=torch.int32, device="cuda")
    out = torch.empty(T, heads, C, dtype=dtype, device="cuda")
    tpt = 16 // min(heads, 16)
    dev = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")
    scale = 0.3
    if kernel.startswith("general"):
        ops.latent_attention(q.cuda(), l_pages, r_pages, bt, torch.zeros(T, dtype=torch.int32, device="cuda"), pos_dev, out,
                             scale, None, window, sinks.cuda())
    elif "many rows" in kernel:
        ops.latent_prefill(q.cuda(), l_pages, r_pages, bt, tuple(dev(x) for x in tile_lists([T], 4 * tpt)), pos_dev, out,
                           scale, None, window, sinks.cuda())
    else:
        ops.latent_flash(q.cuda(), l_pages, r_pages, bt, tuple(dev(x) for x in tile_lists([T], tpt)), pos_dev, out, scale,
                         None, 1, None, window, sinks.cuda())
    rr, lr = torch.cat([lat.to(dtype), kr.to(dtype)], dim=1).double(), lat.to(dtype).double()
    allowed = plain.visible(torch.arange(n), window or None)[n0:]
    got = out.double().cpu()
    for h in range(heads):
        s = (q[:, h].double() @ rr.T) * scale
        want = plain.sink_softmax(s, allowed, sinks[h].double()) @ lr
        assert (got[:, h] - want).abs().max() < (2e-5 if dtype == torch.float32 else 3e-2), h


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("pairing", ["interleaved", "half"])
def test_latent_prepare_without_a_query_latent_and_rotate_into(dtype, pairing):
    """The latent's norm and the shared key part's rotation in either pairing, written at scattered slots (a
    negative slot stores nothing); the queries' rotated part into the float32 query rows."""
    from tiny_llm_amd.kernels import ops
    from tiny_llm_amd.parts.rotary import angle_tables
    g = torch.Generator().manual_seed(2)
    T, C, R, rd, H, D, block, eps = 9, 24, 16, 8, 3, 8, 4, 1e-5
    d = torch.randn(T, 8 + C + R + 8, generator=g).to(dtype)
    wn = 1.0 + 0.2 * torch.randn(C, generator=g)
    positions = torch.randint(0, 300, (T,), generator=g)
    slots = torch.randperm(40, generator=g)[:T].to(torch.int32)
    slots[2] = -1
    cos, sin = angle_tables(rd, 500.0, 512, "cuda")
    latent = torch.full((10, block, C), float("nan"), dtype=dtype, device="cuda")
    rope = torch.full((10, block, R), float("nan"), dtype=dtype, device="cuda")
    ops.latent_prepare(d.cuda(), 0, 0, None, eps, None, 8, C, R, rd, wn.cuda(), positions.to(torch.int32).cuda(), cos, sin,
                       slots.cuda(), latent, rope, pairing)

    def rotate(x):
        if pairing == "interleaved":
            return plain.rotate_pairs(x, positions, rd, 500.0)
        f = 500.0 ** (-2.0 * torch.arange(rd // 2, dtype=torch.float64) / rd)
        ang = positions.double()[:, None] * f[None, :]
        shape = [x.shape[0]] + [1] * (x.dim() - 2) + [rd // 2]
        c, s = torch.cos(ang).reshape(shape), torch.sin(ang).reshape(shape)
        u, v = x[..., :rd // 2], x[..., rd // 2:rd]
        return torch.cat([u * c - v * s, v * c + u * s, x[..., rd:]], dim=-1)

    dd = d.double()
    want_c = plain.rms_norm(dd[:, 8:8 + C], wn.double(), eps)
    want_k = rotate(dd[:, 8 + C:8 + C + R])
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    for t in range(T):
        s = int(slots[t])
        if s >= 0:
            assert (latent[s // block, s % block].double().cpu() - want_c[t]).abs().max() < tol
            assert (rope[s // block, s % block].double().cpu() - want_k[t]).abs().max() < tol
    used = {int(s) for s in slots if s >= 0}
    assert all(torch.isnan(latent[s // block, s % block]).all() for s in range(40) if s not in used)
    q = torch.randn(T, H * (D + R) + 8, generator=g).to(dtype)
    qa = torch.zeros(T, H, C + R, device="cuda")
    ops.rotate_into(q.cuda(), H, D + R, D, R, rd, positions.to(torch.int32).cuda(), cos, sin, qa, C, pairing)
    want_q = rotate(q.double()[:, :H * (D + R)].reshape(T, H, D + R)[:, :, D:])
    assert (qa[:, :, C:].double().cpu() - want_q).abs().max() < 1e-5 and float(qa[:, :, :C].abs().max()) == 0.0


def test_gate_and_activation_rows():
    from tiny_llm_amd.kernels import ops
    g = torch.Generator().manual_seed(0)
    for dtype in (torch.float32, torch.bfloat16):
        wide = torch.randn(7, 50, generator=g).to(dtype).cuda()
        a = torch.randn(7, 24, generator=g).to(dtype).cuda()
        out = ops.gate_rows(a, wide[:, 16:40], torch.empty_like(a))
        want = a.double() * torch.sigmoid(wide[:, 16:40].double())
        assert (out.double() - want).abs().max() < (1e-6 if dtype == torch.float32 else 2e-2)
        x = torch.randn(7, 50, generator=g).cuda()
        z = ops.activate_rows(x[:, 3:43], torch.empty(7, 40, dtype=dtype, device="cuda"), "relu2")
        assert (z.double() - torch.relu(x[:, 3:43].double()) ** 2).abs().max() < (1e-6 if dtype == torch.float32 else 5e-2)
