"""The Gesutar architecture without a GPU: its configuration reader, the model as data, and properties of the
plain implementation (tests/plain_gesutar.py) that the engine is compared with on the GPU."""
import copy
import math

import pytest
import torch

import plain_gesutar as plain
from gesutar_util import CONFIGS, MIX_A, MIX_B, ODD, every_expert, random_config, random_weights
from util import random_tokens


def _decoder(cfg, dtype="float32"):
    from tiny_llm_amd.config import resolve
    from tiny_llm_amd.models.decoder import Decoder
    typed, spec = resolve(cfg)
    return typed, spec, Decoder(spec, dtype=dtype, device="cpu")


def test_reader_takes_every_size_from_the_configuration():
    typed, spec, dec = _decoder(MIX_A)
    assert (typed.vocab, typed.width, typed.norm_eps, typed.embedding_scale) == (301, 64, 1e-5, 3.0)
    assert (typed.bigram.buckets, typed.bigram.mul_prev, typed.bigram.mul_cur) == (97, 7, 13)
    a = typed.layers[1].mixer
    assert (a.heads, a.dim, a.rot_dim, a.vdim, a.kv_rank, a.window, a.rot_dims, a.rot_base, a.scale) == \
        (3, 32, 16, 8, 48, 7, 8, 50000.0, 0.2)
    m = typed.layers[0].mlp
    assert (m.experts, m.top, m.ff, m.groups, m.keep, m.scale, m.shared_ff) == (6, 2, 24, 3, 2, 1.5, 40)
    assert typed.layers[1].mlp.groups == 1 and typed.layers[1].mlp.shared_ff == 0
    assert typed.layers[2].mlp is None and typed.layers[3].mixer.rot_dim == 0
    assert _decoder(MIX_B)[0].layers[2].mixer.window == 0           # no mask: every earlier token is seen
    assert spec.architecture == "Gesutar" and [e.layer for e in spec.plan] == [0, 1, 2, 3]


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_spec_names_the_checkpoints_tensors(name):
    cfg = CONFIGS[name][0]
    _, _, dec = _decoder(cfg)
    want = {k: tuple(v.shape) for k, v in random_weights(cfg).items()}
    got = {w.name: tuple(w.shape) for w in dec.weight_specs()}
    assert got == want


def test_without_a_pair_table_and_without_a_feed_forward():
    from gesutar_util import NO_PAIRS
    typed, spec, dec = _decoder(NO_PAIRS)
    assert typed.bigram is None and spec.embedding.kind == "token_embedding" and dec.embedding.scale == 2.0
    assert dec.state_specs() == {}
    _, spec_a, _ = _decoder(MIX_A)
    assert spec_a.ignorable_tensors == ("l2.norm2",) and "ffn" not in spec_a.layers[2].parts


def test_cache_groups_windows_and_state():
    from tiny_llm_amd.cache import CacheManager
    _, _, dec = _decoder(MIX_A)
    specs = dec.cache_specs()
    assert sorted(specs) == [(i, "mixer") for i in range(4)]
    assert [specs[(i, "mixer")].kind for i in range(4)] == ["window"] * 4
    assert [specs[(i, "mixer")].window for i in range(4)] == [24, 7, 1000, 33]
    assert [t.name for t in specs[(3, "mixer")].tensors] == ["latent"]              # no rotated key part
    assert [t.shape for t in specs[(0, "mixer")].tensors] == [(32,), (8,)]
    assert _decoder(MIX_B)[2].cache_specs()[(2, "mixer")].kind == "full"
    states = dec.state_specs()
    assert list(states) == [dec.EMBEDDING_OWNER] and states[dec.EMBEDDING_OWNER].dtype == torch.int32
    cm = CacheManager(specs, states, 8, 20, 2)
    assert len(cm.groups) == 4
    cm.allocate_tensors(torch.float32, "cpu")
    assert cm.states[dec.EMBEDDING_OWNER].shape == (2, 1)
    # the window of seven gives pages back while the others keep theirs
    cm.reserve_step([("a", 40)])
    cm.commit("a", 40)
    cm.forget_reservation()
    assert cm.free_blocks()[1] > cm.free_blocks()[2]


def test_refusals():
    from tiny_llm_amd.config import ConfigError, resolve

    def broken(change):
        cfg = copy.deepcopy(MIX_A)
        change(cfg)
        with pytest.raises(ConfigError):
            resolve(cfg)

    broken(lambda c: c["layers"][0].update(type="something_else"))
    broken(lambda c: c["layers"][0]["mixer"].pop("kv_rank"))
    broken(lambda c: c["layers"][0]["mixer"].pop("scale"))
    broken(lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7))
    broken(lambda c: c["layers"][0]["mixer"]["rot"].update(dims=10))            # more than rot_dim
    broken(lambda c: c["layers"][0]["mlp"]["router"].update(top=7))             # more than experts
    broken(lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=4))  # does not divide 6
    broken(lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(keep=1, count=3) or
           c["layers"][0]["mlp"]["router"].update(top=3))                       # one group holds two experts
    broken(lambda c: c["layers"][0]["mlp"].update(kind="dense"))
    broken(lambda c: c["embedding"]["bigram"].pop("mul_cur"))
    broken(lambda c: c.pop("norm"))
    with pytest.raises(ConfigError):
        cfg = copy.deepcopy(MIX_A)
        resolve(cfg, {"bigram": (50, 64)})                                      # the table's rows are not buckets + 1
    with pytest.raises(Exception):
        cfg = copy.deepcopy(MIX_A)
        cfg["layers"][0]["mixer"]["kv_rank"] = 20                               # bfloat16 needs multiples of 8
        _decoder(cfg, "bfloat16")


def test_sizes_the_bfloat16_kernels_refuse_are_served_in_float32():
    """The front ends' builder: a bfloat16 engine given a model with rows of no multiple of 8 elements builds
    the float32 decoder and warns, naming the size; sizes that both refuse are refused; a model that fits is
    built as asked."""
    from tiny_llm_amd.engine.loading import build_decoder
    from tiny_llm_amd.kernels.ops import KernelError
    with pytest.warns(RuntimeWarning, match="served in float32.*hidden_size = 50"):
        _, dec = build_decoder(ODD, "bfloat16", "cpu")
    assert dec.dtype == torch.float32
    cfg = copy.deepcopy(MIX_A)
    cfg["layers"][0]["mlp"]["expert"]["ff"] = 20
    with pytest.warns(RuntimeWarning, match="intermediate_size = 20"):
        assert build_decoder(cfg, "bfloat16", "cpu")[1].dtype == torch.float32
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        assert build_decoder(MIX_A, "bfloat16", "cpu")[1].dtype == torch.bfloat16
        assert build_decoder(ODD, "float32", "cpu")[1].dtype == torch.float32
    cfg = copy.deepcopy(MIX_A)
    cfg["layers"][0]["mixer"]["kv_rank"] = 100000
    for dtype in ("bfloat16", "float32"):
        with pytest.raises(KernelError):
            build_decoder(cfg, dtype, "cpu")


def test_configurations_drawn_at_random_build():
    for seed in range(30):
        cfg = random_config(seed)
        _, _, dec = _decoder(cfg, "bfloat16")
        assert {w.name for w in dec.weight_specs()} == set(random_weights(cfg))


# ------------------------------------------------------------------ the plain implementation
def test_bigram_rows():
    rows = plain.bigram_rows([5, 9, 9, 0], 7, 3, 10)
    assert rows.tolist() == [7, (5 * 3 + 9 * 10) % 7, (9 * 3 + 9 * 10) % 7, (9 * 3) % 7]
    assert plain.bigram_rows([4], 1, 1, 1).tolist() == [1]


def test_embedding_depends_on_the_token_before():
    cfg = MIX_A
    w = {k: v.double() for k, v in random_weights(cfg).items()}
    a = plain.embed([3, 8, 20], w, cfg["embedding"])
    b = plain.embed([4, 8, 20], w, cfg["embedding"])
    assert not torch.allclose(a[1], b[1]) and torch.allclose(a[2], b[2])
    assert torch.allclose(a[0], w["embed"][3] * 3.0 + w["bigram"][97])


def test_sink_takes_weight_and_window_hides_keys():
    s = torch.tensor([[0.5, -1.0, 2.0]], dtype=torch.float64)
    ok = torch.ones(1, 3, dtype=torch.bool)
    p = plain.sink_softmax(s, ok, torch.tensor(1.0, dtype=torch.float64))
    z = math.exp(1.0) + sum(math.exp(v) for v in (0.5, -1.0, 2.0))
    assert torch.allclose(p, torch.tensor([[math.exp(0.5) / z, math.exp(-1.0) / z, math.exp(2.0) / z]], dtype=torch.float64))
    assert plain.sink_softmax(s, ok, torch.tensor(50.0, dtype=torch.float64)).sum() < 1e-15
    assert abs(float(plain.sink_softmax(s, ok, torch.tensor(-50.0, dtype=torch.float64)).sum()) - 1) < 1e-15
    pos = torch.arange(6)
    vis = plain.visible(pos, 3)
    assert vis[5].tolist() == [False, False, False, True, True, True] and vis[1].tolist() == [True, True] + [False] * 4
    assert plain.visible(pos, None)[5].all()


def test_a_token_outside_every_window_reaches_nothing():
    """Windows of 24, 7 and 33 and one longer than the prompt in layer 2: with that layer's window cut to 9, the
    first token of a long prompt cannot reach the last logits through any path of four layers."""
    cfg = copy.deepcopy(MIX_A)
    cfg["layers"][2]["mixer"]["mask"]["size"] = 9
    w = {k: v.double() for k, v in random_weights(cfg, 4).items()}
    toks = random_tokens(90, cfg["vocab"], 3)
    other = list(toks)
    other[0] = (toks[0] + 1) % cfg["vocab"]
    a, b = plain.forward(cfg, w, toks), plain.forward(cfg, w, other)
    reach = 1 + (24 - 1) + (7 - 1) + (9 - 1) + (33 - 1)            # token 1 carries token 0 in its bigram row
    assert torch.equal(a[reach + 1:], b[reach + 1:]) and not torch.equal(a[:reach], b[:reach])


def test_router():
    z = torch.tensor([[2.0, 0.1, 0.0, 1.9, 3.0, -5.0]], dtype=torch.float64)
    s = torch.softmax(z, -1)[0]
    idx, wts = plain.route(z, {"experts": 6, "top": 2, "scale": 1.5})
    assert idx.tolist() == [[4, 0]]
    assert torch.allclose(wts[0], torch.stack([s[4], s[0]]) / (s[4] + s[0]) * 1.5)
    # three groups of two, the best two kept: groups score 2.0, 1.9 and 3.0, so experts 2 and 3 are out
    idx, _ = plain.route(z, {"experts": 6, "top": 3, "groups": {"count": 3, "keep": 2}})
    assert sorted(idx[0].tolist()) == [0, 1, 4]
    idx, _ = plain.route(z, {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 1}})
    assert sorted(idx[0].tolist()) == [4, 5]
    idx, wts = plain.route(z, {"experts": 6, "top": 6})
    assert abs(float(wts.sum()) - 1.0) < 1e-12


def test_every_expert_variant_weighs_by_score():
    cfg = every_expert(MIX_A)
    assert [l["mlp"]["router"]["top"] for l in cfg["layers"] if l["mlp"]] == [6, 4, 8]
    w = {k: v.double() for k, v in random_weights(ODD, 1).items()}
    logits = plain.forward(ODD, w, random_tokens(20, ODD["vocab"], 0))
    assert logits.shape == (20, ODD["vocab"]) and torch.isfinite(logits).all()
