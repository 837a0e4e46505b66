"""The Vevapel architecture without a GPU: its configuration reader, the model as data (the plan of a repeated run
of layers, caches and states of every pass), and properties of the plain implementation (tests/plain_vevapel.py)
that the engine is compared with on the GPU."""
import copy
import math

import pytest
import torch

import plain_vevapel as plain
from vevapel_util import CONFIGS, LOOP_ALL, LOOP_ONE, MIX_A, MIX_B, ODD, every_expert, random_config, random_weights
from util import random_tokens


def _decoder(cfg, dtype="float32"):
    from tiny_llm_amd.config import resolve
    from tiny_llm_amd.models.decoder import Decoder
    typed, spec = resolve(cfg)
    return typed, spec, Decoder(spec, dtype=dtype, device="cpu")


def test_reader_takes_every_size_from_the_configuration():
    typed, spec, dec = _decoder(MIX_A)
    assert (typed.vocab, typed.width, typed.norm_eps, typed.embedding_scale, typed.residual_mult) == (301, 64, 1e-5, 2.5, 0.6)
    a = typed.layers[0].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.temp_coef, a.temp_every, a.scale) == (4, 2, 24, 16, 0.4, 16, 2.0 * 24 ** -0.5)
    d = typed.layers[1].mixer
    assert (d.heads, d.kv_heads, d.dim, d.vdim, d.conv) == (4, 2, 16, 8, 4)
    b = typed.layers[5].mixer
    assert (b.heads, b.kv_heads, b.dim, b.vdim, b.diff, b.chunk, b.rot_dims, b.rot_base) == (2, 1, 32, 16, 0.6, 7, 32, 40000.0)
    m = typed.layers[0].mlp
    assert (m.experts, m.top, m.ff) == (6, 2, 24) and typed.layers[2].mlp is None
    assert (typed.loop.start, typed.loop.stop, typed.loop.times) == (1, 4, 3)
    tb = _decoder(MIX_B)[0]
    assert tb.loop is None and tb.layers[2].mixer.temp_every == 0           # no temperature
    assert tb.layers[4].mixer.chunk == 0 and tb.layers[3].mixer.rot_dims == 0  # no mask, no rotation
    assert spec.architecture == "Vevapel"
    assert dec.layers[0].block.mult == 0.6 and dec.embedding.scale == 2.5


def test_plan_of_a_repeated_run():
    """Layers start .. stop - 1 run `times` times in a row; every run is a plan entry of its own (caches and
    states of its own), and the first run of every pass is entered through the stream part."""
    _, spec, dec = _decoder(MIX_A)
    assert [e.layer for e in spec.plan] == [0, 1, 2, 3, 1, 2, 3, 1, 2, 3, 4, 5]
    assert [e.before for e in spec.plan] == [None, (0, 0), None, None, (0, 1), None, None, (0, 2), None, None, None, None]
    assert all(e.cache_of is None for e in spec.plan)
    assert [p.kind for p in spec.stream_parts] == ["loop_join"] and dec.stream_parts[0].times == 3
    _, spec_all, _ = _decoder(LOOP_ALL)
    assert [(e.layer, e.before) for e in spec_all.plan] == [(0, (0, 0)), (1, None)]
    _, spec_one, _ = _decoder(LOOP_ONE)
    assert [e.layer for e in spec_one.plan] == [0, 1, 1, 1, 1, 1, 2]
    assert [e.before for e in spec_one.plan][1:6] == [(0, t) for t in range(5)]
    _, spec_b, dec_b = _decoder(MIX_B)
    assert spec_b.stream_parts == () and dec_b.stream_parts == [] and all(e.before is None for e in spec_b.plan)
    assert [(i, first) for i, _, first in plain.run_order(MIX_A)] == [(e.layer, e.before is not None) for e in spec.plan]
    assert [t for _, t, first in plain.run_order(MIX_A) if first] == [e.before[1] for e in spec.plan if e.before]


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_spec_names_the_checkpoints_tensors(name):
    cfg = CONFIGS[name][0]
    _, _, dec = _decoder(cfg)
    want = {k: tuple(v.shape) for k, v in random_weights(cfg).items()}
    got = {w.name: tuple(w.shape) for w in dec.weight_specs() if not w.alias_of}
    assert got == want
    tied = [w for w in dec.weight_specs() if w.alias_of]
    assert [(w.name, w.alias_of) for w in tied] == [("head", "embed")]       # the head is the embedding table


def test_cache_groups_and_states_of_every_pass():
    from tiny_llm_amd.cache import CacheManager
    _, spec, dec = _decoder(MIX_A)
    specs = dec.cache_specs()
    # attention layers 0, 3 and 5, differential layer 2; layers 2 and 3 run three times
    assert sorted(i for i, _ in specs) == [0, 2, 3, 5, 6, 8, 9, 11]
    assert [t.name for t in specs[(2, "mixer")].tensors] == ["k", "k2", "v"]        # two maps share the values
    assert [t.name for t in specs[(0, "mixer")].tensors] == ["k", "v"]
    # heads of 24 keys and 16 values lie in rows of 32; 16 and 24 in rows of 32; 8 and 40 in rows of 48
    assert [specs[(i, "mixer")].tensors[0].shape for i in (0, 2, 3, 11)] == [(2, 32), (2, 32), (3, 48), (1, 32)]
    assert all(s.kind == "full" for s in specs.values())
    states = dec.state_specs()
    assert sorted(i for i, _ in states) == [1, 4, 7, 10]                             # the delta layers' runs
    d = dec.layers[1].mixer
    assert states[(1, "mixer")].shape == (4 * 16 * 8 + (2 * 2 * 16 + 4 * 8) * 3,) and d.per_head and d.direct
    cm = CacheManager(specs, states, 8, 20, 2)
    cm.allocate_tensors(torch.float32, "cpu")
    assert len({id(cm.states[k]) for k in states}) == 4                              # a state of its own per pass


def test_refusals():
    from tiny_llm_amd.config import ConfigError, resolve

    def broken(change, base=MIX_A):
        cfg = copy.deepcopy(base)
        change(cfg)
        with pytest.raises(ConfigError):
            resolve(cfg)

    broken(lambda c: c["layers"][0].update(type="something_else"))
    broken(lambda c: c["layers"][0]["mixer"].pop("scale"))
    broken(lambda c: c["layers"][0]["mixer"].pop("vdim"))
    broken(lambda c: c["layers"][0]["mixer"].update(heads=3))                    # no multiple of kv_heads
    broken(lambda c: c["layers"][0]["mixer"]["q_temp"].update(every=0))
    broken(lambda c: c["layers"][1]["mixer"].pop("conv"))
    broken(lambda c: c["layers"][2]["mixer"]["rot"].update(dims=7))
    broken(lambda c: c["layers"][2]["mixer"]["rot"].update(dims=18))             # more than dim
    broken(lambda c: c["layers"][2]["mixer"].pop("diff"))
    broken(lambda c: c["layers"][0]["mlp"]["router"].update(top=7))              # more than experts
    broken(lambda c: c["layers"][0]["mlp"].update(kind="dense"))
    broken(lambda c: c["loop"].update(stop=7))                                   # beyond the layers
    broken(lambda c: c["loop"].update(start=4))                                  # an empty run
    broken(lambda c: c["loop"].update(times=0))
    broken(lambda c: c.pop("norm"))
    with pytest.raises(ConfigError):
        resolve(copy.deepcopy(MIX_A), {"loop.step": (2, 64)})                    # a vector per pass


def test_sizes_the_bfloat16_kernels_refuse_are_served_in_float32():
    from tiny_llm_amd.engine.loading import build_decoder
    with pytest.warns(RuntimeWarning, match="served in float32"):
        _, dec = build_decoder(ODD, "bfloat16", "cpu")
    assert dec.dtype == torch.float32
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        assert build_decoder(MIX_A, "bfloat16", "cpu")[1].dtype == torch.bfloat16


def test_configurations_drawn_at_random_build():
    for seed in range(30):
        cfg = random_config(seed)
        _, _, dec = _decoder(cfg, "bfloat16")
        assert {w.name for w in dec.weight_specs() if not w.alias_of} == set(random_weights(cfg))


# ------------------------------------------------------------------ the plain implementation
def test_layer_norm_and_unit_rms():
    x = torch.tensor([[1.0, 2.0, 3.0, 6.0]], dtype=torch.float64)
    w, b = torch.tensor([1.0, 2.0, 1.0, 0.5], dtype=torch.float64), torch.tensor([0.0, 1.0, 0.0, 0.0], dtype=torch.float64)
    mu, var = 3.0, (4 + 1 + 0 + 9) / 4
    want = (x - mu) / math.sqrt(var + 1e-5) * w + b
    assert torch.allclose(plain.layer_norm(x, w, b, 1e-5), want)
    assert torch.allclose(plain.unit_rms(x, 0.0), x / math.sqrt((1 + 4 + 9 + 36) / 4))


def test_masks():
    pos = torch.arange(10)
    ch = plain.same_chunk(pos, 4)
    assert ch[5].tolist() == [False] * 4 + [True, True] + [False] * 4             # chunk 4..7, causal
    assert ch[4].tolist() == [False] * 4 + [True] + [False] * 5                   # a chunk's first token sees itself
    assert ch[3].tolist() == [True] * 4 + [False] * 6
    assert plain.causal(pos)[3].tolist() == [True] * 4 + [False] * 6
    # a chunk begins at a multiple of its size whatever the first position given is
    assert plain.same_chunk(torch.arange(6, 9), 4)[2].tolist() == [False, False, True]


def test_query_temperature():
    pos = torch.tensor([0, 14, 15, 16, 47, 48])
    t = plain.query_temperature(pos, 0.5, 16)
    want = [1.0, 1.0, 1 + 0.5 * math.log(2), 1 + 0.5 * math.log(2), 1 + 0.5 * math.log(4), 1 + 0.5 * math.log(4)]
    assert torch.allclose(t, torch.tensor(want, dtype=torch.float64))


def test_rotation_pairs_halves_and_leaves_the_rest():
    x = torch.arange(1.0, 9.0, dtype=torch.float64).reshape(1, 1, 8)
    y = plain.rotate_half(x, torch.tensor([3]), 4, 100.0)
    f = [1.0, 100.0 ** -0.5]
    for i in range(2):
        a = 3 * f[i]
        assert abs(float(y[0, 0, i]) - (x[0, 0, i] * math.cos(a) - x[0, 0, i + 2] * math.sin(a))) < 1e-12
        assert abs(float(y[0, 0, i + 2]) - (x[0, 0, i + 2] * math.cos(a) + x[0, 0, i] * math.sin(a))) < 1e-12
    assert torch.equal(y[..., 4:], x[..., 4:])
    assert torch.equal(plain.rotate_half(x, torch.tensor([0]), 8, 100.0), x)


def test_router_weighs_the_chosen_logits_alone():
    h = torch.eye(3, dtype=torch.float64)
    w_r = torch.tensor([[2.0, 0.0, 0.5], [0.1, 5.0, 0.0], [0.0, 0.0, -1.0], [1.9, 4.0, 0.0]], dtype=torch.float64)
    b = torch.tensor([0.0, 0.0, 3.0, 0.0], dtype=torch.float64)
    ids, wts = plain.route(h, w_r, b, 2)
    z = h @ w_r.T + b
    assert ids.tolist() == [[2, 0], [1, 3], [2, 0]]
    for t in range(3):
        chosen = z[t, ids[t]]
        assert torch.allclose(wts[t], torch.exp(chosen) / torch.exp(chosen).sum())
    assert abs(float(plain.route(h, w_r, b, 4)[1][0].sum()) - 1.0) < 1e-12


def test_short_convolution_starts_from_zeros():
    x = torch.arange(1.0, 6.0, dtype=torch.float64).reshape(5, 1)
    taps = torch.tensor([[0.5, -1.0, 2.0]], dtype=torch.float64)            # the last column is the current token's
    y = plain.short_conv(x, taps)
    assert y[:, 0].tolist() == [2.0, 2.0 * 2 - 1.0, 2.0 * 3 - 2.0 + 0.5, 2.0 * 4 - 3.0 + 1.0, 2.0 * 5 - 4.0 + 1.5]


def test_delta_scan_against_its_closed_form():
    """With beta = 1, no decay and orthonormal keys the state holds each key's value exactly: o_t = sum over the
    keys seen so far of (q_t . k_j) v_j, and a repeated key replaces its value."""
    D, V = 4, 3
    k = torch.eye(D, dtype=torch.float64)[[0, 1, 0, 2]].reshape(4, 1, D)
    v = torch.arange(12, dtype=torch.float64).reshape(4, 1, V)
    q = torch.ones(4, 1, D, dtype=torch.float64)
    o = plain.delta_scan(q, k, v, torch.ones(4, 1, dtype=torch.float64), torch.ones(4, 1, dtype=torch.float64))
    assert torch.allclose(o[1, 0], v[0, 0] + v[1, 0])
    assert torch.allclose(o[2, 0], v[2, 0] + v[1, 0])                        # key 0 written again
    assert torch.allclose(o[3, 0], v[2, 0] + v[1, 0] + v[3, 0])
    # a decay of one half per token on what was written before, read in the same step as the write
    g = torch.full((4, 1), 0.5, dtype=torch.float64)
    o = plain.delta_scan(q, k, v, torch.ones(4, 1, dtype=torch.float64), g)
    assert torch.allclose(o[1, 0], 0.5 * v[0, 0] + v[1, 0])


def test_a_token_outside_the_chunk_reaches_later_logits_only_through_other_layers():
    """One differential layer alone with chunks of 20: the last chunk's logits do not change with a token of an
    earlier chunk; with a delta layer in front they do (its state carries everything)."""
    cfg = CONFIGS["diff"][0]
    w = {k: v.double() for k, v in random_weights(cfg, 4).items()}
    toks = random_tokens(50, cfg["vocab"], 3)
    other = list(toks)
    other[5] = (toks[5] + 1) % cfg["vocab"]
    a, b = plain.forward(cfg, w, toks), plain.forward(cfg, w, other)
    assert torch.equal(a[20:], b[20:]) and not torch.equal(a[5:20], b[5:20])
    both = copy.deepcopy(cfg)
    both["layers"] = [CONFIGS["delta"][0]["layers"][0]] + cfg["layers"]
    w2 = {k: v.double() for k, v in random_weights(both, 4).items()}
    a, b = plain.forward(both, w2, toks), plain.forward(both, w2, other)
    assert not torch.equal(a[40:], b[40:])


def test_every_pass_adds_its_own_vector():
    cfg = LOOP_ONE
    w = {k: v.double() for k, v in random_weights(cfg, 2).items()}
    toks = random_tokens(12, cfg["vocab"], 1)
    base = plain.forward(cfg, w, toks)
    for t in range(cfg["loop"]["times"]):
        w2 = dict(w)
        w2["loop.step"] = w["loop.step"].clone()
        w2["loop.step"][t, 0] += 1.0           # (one channel: a shift of every channel alike is what a layer norm removes)
        assert not torch.allclose(plain.forward(cfg, w2, toks), base)
    trace = []
    plain.forward(cfg, w, toks, trace=trace)
    assert len(trace) == 7


def test_every_expert_variant():
    cfg = every_expert(MIX_A)
    assert [l["mlp"]["router"]["top"] for l in cfg["layers"] if l["mlp"]] == [6, 4, 8, 3, 5]
    w = {k: v.double() for k, v in random_weights(ODD, 1).items()}
    logits = plain.forward(ODD, w, random_tokens(20, ODD["vocab"], 0))
    assert logits.shape == (20, ODD["vocab"]) and torch.isfinite(logits).all()
