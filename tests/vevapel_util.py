"""Test material for the Vevapel architecture: small configurations that differ from each other in every size
and option, and a generator of random checkpoints for them (numpy, its own scales: queries and keys that make
the softmax far from uniform, decays that forget at a visible rate, routers that decide, biases and norm
weights that are neither zero nor one)."""
import copy
import json
import os

import numpy as np
import torch

from fofapel_util import as_double, rounded, row_err  # noqa: F401  (the same comparisons serve every design)


def attention(heads, kv_heads, dim, vdim, q_temp=(0.4, 16), scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
         "scale": float(scale if scale is not None else 2.0 * dim ** -0.5)}
    if q_temp:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return {"type": "attention", "mixer": m}


def attention_2(heads, kv_heads, dim, vdim, chunk, rot_dims, diff=0.25, base=10000.0, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": diff,
         "scale": float(scale if scale is not None else 2.0 * dim ** -0.5)}
    if chunk:
        m["mask"] = {"size": chunk}
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
    return {"type": "attention_2", "mixer": m}


def delta(heads, kv_heads, dim, vdim, conv):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def moe(experts, top, ff):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}


def layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


def model(width, vocab, layers, loop=None, mult=0.6, scale=2.5, eps=1e-5):
    cfg = {"architecture": "Vevapel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult,
           "embedding": {"scale": scale}, "layers": layers}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


# every mixer, sizes that differ from layer to layer: keys wider and narrower than values, grouped and ungrouped heads,
# chunks of 24 and 7 positions and none, part and all of a map rotated, temperatures that step every 16 and every 5
# positions, 2 to 4 taps, a layer without feed-forward; layers 1 to 3 run three times
MIX_A = model(64, 301, [
    layer(attention(4, 2, 24, 16, (0.4, 16)), moe(6, 2, 24)),
    layer(delta(4, 2, 16, 8, 4), moe(4, 1, 16)),
    layer(attention_2(4, 2, 16, 24, 24, 8, 0.35, 1000.0), None),
    layer(attention(3, 3, 8, 40, (1.5, 5)), moe(8, 3, 8)),
    layer(delta(2, 2, 32, 16, 2), moe(3, 3, 16)),
    layer(attention_2(2, 1, 32, 16, 7, 32, 0.6, 40000.0), moe(5, 2, 8)),
], loop=(1, 4, 3))

# no loop; one head, twenty heads (two tiles of heads), a chunk of one position (a token sees itself alone), a chunk
# longer than any prompt, no mask, no rotation, no temperature, three taps, one expert, every expert, a multiplier of one
MIX_B = model(128, 257, [
    layer(attention_2(1, 1, 64, 128, 1, 64, 0.1), moe(2, 2, 32)),
    layer(delta(8, 1, 16, 16, 3), moe(1, 1, 16)),
    layer(attention(20, 4, 8, 8, None), None),
    layer(attention_2(8, 8, 16, 8, 1000, 0, 0.5), moe(9, 3, 8)),
    layer(attention_2(6, 3, 8, 16, 0, 4, 0.2, 100.0), moe(5, 5, 16)),
    layer(delta(3, 3, 24, 40, 4), None),
], loop=None, mult=1.0, scale=1.0, eps=3e-6)

# the whole model is one repeated run (the pass begins at the first layer), once; and a run of one layer five times
LOOP_ALL = model(64, 199, [layer(attention(2, 1, 16, 16, (0.3, 7)), moe(4, 2, 16)), layer(delta(2, 1, 16, 16, 4), None)],
                 loop=(0, 2, 1))
LOOP_ONE = model(64, 199, [layer(delta(2, 2, 16, 8, 4), moe(3, 1, 8)), layer(attention_2(2, 2, 16, 16, 10, 16), moe(4, 2, 16)),
                           layer(attention(4, 1, 16, 8, (0.6, 9)), None)], loop=(1, 2, 5), mult=0.4)

# sizes that are multiples of nothing (float32 only)
ODD = model(50, 199, [
    layer(attention(3, 1, 10, 7, (0.7, 3)), moe(5, 2, 11)),
    layer(delta(3, 1, 5, 9, 3), moe(6, 4, 3)),
    layer(attention_2(2, 2, 6, 11, 13, 4, 0.25, 777.0), moe(2, 1, 7)),
], loop=(0, 2, 2), scale=0.5)

# heads beyond what the matrix-core attention kernels take: the general kernel in both precisions
WIDE = model(64, 199, [layer(attention(2, 1, 136, 200, (0.3, 11)), moe(3, 2, 16)),
                       layer(attention_2(2, 2, 40, 144, 33, 20, 0.4), None)], loop=(1, 2, 2))

ONLY_ATTENTION = model(64, 199, [layer(attention(6, 2, 16, 8, (0.8, 8)), None)])
ONLY_DIFF = model(64, 199, [layer(attention_2(4, 2, 16, 24, 20, 8), None)])
ONLY_DELTA = model(64, 199, [layer(delta(4, 2, 16, 24, 4), None)])
ONLY_MOE = model(64, 199, [layer(attention(2, 2, 8, 8, None), moe(8, 3, 16))])

CONFIGS = {"A": (MIX_A, 16), "B": (MIX_B, 8), "loop_all": (LOOP_ALL, 4), "loop_one": (LOOP_ONE, 16), "odd": (ODD, 4),
           "wide": (WIDE, 16), "attention": (ONLY_ATTENTION, 4), "diff": (ONLY_DIFF, 8), "delta": (ONLY_DELTA, 16), "moe": (ONLY_MOE, 16)}


def every_expert(cfg):
    """The same model with every expert chosen by every token: its routing cannot flip where two logits are
    close, so a bfloat16 engine and the plain model choose alike."""
    out = copy.deepcopy(cfg)
    for l in out["layers"]:
        if l["mlp"]:
            l["mlp"]["router"]["top"] = l["mlp"]["router"]["experts"]
    return out


def tame(cfg, mult=0.3):
    """The model a bfloat16 engine is compared on: every expert chosen by every token, and a sublayer's normed result
    added times at most `mult`.  A norm sits behind every sublayer, so a sublayer's relative rounding error reaches
    the stream undamped, times the multiplier; at 0.6 and more, twelve layer runs nearly double it from run to run
    (rounding nothing but the sublayers' inputs to bfloat16 moves a row of the plain model by up to 1.2e-1), at 0.3 they
    do not (1.7e-2)."""
    out = every_expert(cfg)
    out["residual_mult"] = min(out.get("residual_mult", 1.0), mult)
    return out


def random_config(seed, multiple=8):
    """A configuration drawn at random: width, vocabulary, constants, two to five layers that each draw their own
    mixer, head counts and sizes, and a loop over some run of them (or none)."""
    import random
    rng = random.Random(seed)
    m = multiple
    width = rng.choice([64, 96, 128, 192, 256])
    layers = []
    for _ in range(rng.randrange(2, 6)):
        kv = rng.choice([1, 2, 3, 4])
        heads = kv * rng.choice([1, 2, 4])
        dim, vdim = m * rng.randrange(1, 9), m * rng.randrange(1, 9)
        kind = rng.choice(["attention", "attention_2", "delta"])
        if kind == "attention":
            mix = attention(heads, kv, dim, vdim, rng.choice([None, (0.4, 32), (1.0, 3), (0.2, 1)]))
        elif kind == "attention_2":
            mix = attention_2(heads, kv, dim, vdim, rng.choice([0, 1, 2, 5, 16, 31, 64, 100, 5000]),
                              rng.choice([0, dim, max(2, dim // 2 // 2 * 2)]), rng.choice([0.1, 0.35, 0.8]),
                              rng.choice([100.0, 10000.0, 250000.0]))
        else:
            mix = delta(heads, kv, dim, vdim, rng.choice([2, 3, 4]))
        mlp = None
        if rng.random() < 0.75:
            e = rng.randrange(1, 10)
            mlp = moe(e, rng.randrange(1, e + 1), m * rng.randrange(1, 12))
        layers.append(layer(mix, mlp))
    loop = None
    if rng.random() < 0.7:
        start = rng.randrange(0, len(layers))
        loop = (start, rng.randrange(start + 1, len(layers) + 1), rng.randrange(1, 4))
    return model(width, rng.randrange(90, 700), layers, loop, mult=rng.choice([1.0, 0.6, 0.3]),
                 scale=rng.choice([1.0, 4.0, 11.0]), eps=rng.choice([1e-5, 1e-6, 1e-4]))


def random_weights(cfg, seed=0, sharpen=3.0):
    """{name: tensor} (float32).  `sharpen`: the gain of the projections that make scores and gates (3: far from
    uniform, a misplaced key or a lost state moves the logits; 1: tame, so that bfloat16 rounding is not amplified)."""
    lively = 2.0 if sharpen > 1.0 else 1.0
    rng = np.random.default_rng(seed)
    W, V, out = cfg["width"], cfg["vocab"], {}

    def mat(name, rows, cols, gain=1.0):
        out[name] = rng.standard_normal((rows, cols)) * gain / np.sqrt(cols)

    def vec(name, n, mean=0.0, std=0.1):
        out[name] = mean + std * rng.standard_normal(n)

    def norm(name):
        vec(name, W, 1.0, 0.2)
        vec(name + ".b", W, 0.0, 0.2)

    mat("embed", V, W, gain=np.sqrt(W) / max(cfg["embedding"].get("scale", 1.0), 1.0))
    if cfg.get("loop"):
        mat("loop.in", W, 2 * W, gain=1.2)
        out["loop.step"] = 0.5 * rng.standard_normal((cfg["loop"]["times"], W))
    for i, l in enumerate(cfg["layers"]):
        p, a = f"l{i}.", l["mixer"]
        H, G, D, Vd = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
        norm(p + "norm1")
        norm(p + "norm1b")
        if l["type"] == "attention":
            mat(p + "mix.q", H * D, W, gain=sharpen)
            mat(p + "mix.k", G * D, W, gain=sharpen)
            mat(p + "mix.v", G * Vd, W)
            for n, size in (("q", H * D), ("k", G * D), ("v", G * Vd)):
                vec(p + f"mix.{n}.b", size, 0.0, 0.3)
            vec(p + "mix.q.norm", H * D, 1.0, 0.3)
            vec(p + "mix.k.norm", G * D, 1.0, 0.3)
            mat(p + "mix.g", H, W, gain=lively)
            mat(p + "mix.o", W, H * Vd)
            vec(p + "mix.o.b", W, 0.0, 0.3)
        elif l["type"] == "attention_2":
            mat(p + "mix.q", H * 2 * D, W, gain=sharpen)
            mat(p + "mix.k", G * 2 * D, W, gain=sharpen)
            mat(p + "mix.v", G * Vd, W)
            for n, size in (("q", H * 2 * D), ("k", G * 2 * D), ("v", G * Vd)):
                vec(p + f"mix.{n}.b", size, 0.0, 0.3)
            for n in ("lq1", "lk1", "lq2", "lk2"):
                vec(p + f"mix.{n}", D, 0.0, 0.6 / np.sqrt(D) ** 0.5)
            mat(p + "mix.g", H * Vd, W, gain=lively)
            mat(p + "mix.o", W, H * Vd)
        else:
            taps = a["conv"]
            mat(p + "mix.q", G * D, W, gain=sharpen)
            mat(p + "mix.k", G * D, W, gain=sharpen)
            mat(p + "mix.v", H * Vd, W, gain=lively)
            for n, size in (("q", G * D), ("k", G * D), ("v", H * Vd)):
                out[p + f"mix.{n}.conv"] = rng.standard_normal((size, taps)) * 0.6
            mat(p + "mix.b", H, W, gain=lively)
            mat(p + "mix.a", H, W, gain=lively)
            vec(p + "mix.A_log", H, -0.5, 0.7)
            vec(p + "mix.dt_bias", H, 0.0, 0.7)
            vec(p + "mix.norm", Vd, 1.0, 0.2)
            mat(p + "mix.g", H * Vd, W, gain=lively)
            mat(p + "mix.o", W, H * Vd)
        mlp = l["mlp"]
        if mlp is not None:
            norm(p + "norm2")
            norm(p + "norm2b")
            F = mlp["expert"]["ff"]
            for e in range(mlp["router"]["experts"]):
                mat(p + f"mlp.e{e}.gate", F, W, gain=lively)
                mat(p + f"mlp.e{e}.up", F, W, gain=lively)
                mat(p + f"mlp.e{e}.down", W, F)
            mat(p + "mlp.router", mlp["router"]["experts"], W, gain=2.0 * lively)
            vec(p + "mlp.router.b", mlp["router"]["experts"], 0.0, 0.5)
    norm("final.norm")
    return {k: torch.from_numpy(np.asarray(v, dtype=np.float32)) for k, v in out.items()}


def make_folder(path, cfg, seed=0, store=torch.float32, sharpen=3.0):
    """config.json and model.safetensors (written with the safetensors library).  Returns (folder, weights)."""
    from safetensors.torch import save_file
    folder = str(path)
    os.makedirs(folder, exist_ok=True)
    w = random_weights(cfg, seed, sharpen)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(store).contiguous() for k, v in w.items()}, os.path.join(folder, "model.safetensors"))
    return folder, w
