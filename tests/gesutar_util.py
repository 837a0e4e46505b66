"""Test material for the Gesutar architecture: small configurations that differ from each other in every
size and option, and a generator of random checkpoints for them (numpy, its own scales: queries and keys
that make the softmax far from uniform, sinks of both signs, routers that decide, norm weights that are not
one)."""
import copy
import json
import os

import numpy as np
import torch

from fofapel_util import as_double, rounded, row_err  # noqa: F401  (the same comparisons serve every design)


def mixer(heads, dim, rot_dim, vdim, kv_rank, window, rot_dims=None, base=10000.0, scale=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
         "scale": float(scale if scale is not None else 2.0 * (dim + rot_dim) ** -0.5)}
    if window:
        m["mask"] = {"size": window}
    if rot_dim:
        m["rot"] = {"base": base, "dims": rot_dims if rot_dims is not None else rot_dim}
    return m


def moe(experts, top, ff, groups=None, scale=1.0, shared=None):
    r = {"experts": experts, "top": top, "scale": scale}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    m = {"kind": "moe", "router": r, "expert": {"ff": ff}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def layer(m, mlp):
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def model(width, vocab, layers, bigram=(97, 7, 13), scale=3.0, eps=1e-5):
    emb = {"scale": scale}
    if bigram:
        emb["bigram"] = {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}
    return {"architecture": "Gesutar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": emb, "layers": layers}


# windows, head shapes, latents and rotated dims that differ from layer to layer (four cache groups); fewer
# rotated dims than the key part has, none at all; twenty heads (two tiles of heads), a latent that is no
# multiple of 16 (the general kernel in bfloat16); a window longer than any prompt; groups of which some and
# all are kept, no groups, one expert a token, no shared expert, a layer without feed-forward
MIX_A = model(64, 301, [
    layer(mixer(4, 16, 8, 24, 32, 24, 8, 1000.0, 0.3), moe(6, 2, 24, (3, 2), 1.5, 40)),
    layer(mixer(3, 32, 16, 8, 48, 7, 8, 50000.0, 0.2), moe(4, 1, 16, None, 1.0, None)),
    layer(mixer(20, 8, 8, 8, 16, 1000, 8, 100.0), None),
    layer(mixer(2, 24, 0, 16, 40, 33), moe(8, 3, 8, (4, 4), 2.5, 16)),
])

# one bucket, multipliers of one, no scale; a window of one token (a token sees itself and the sink), one head,
# values wider than the stream; a layer without mask (every earlier token is seen) and without feed-forward;
# every expert used by every token; one group kept; sixteen heads
MIX_B = model(128, 257, [
    layer(mixer(1, 64, 64, 128, 64, 1, 64, 250.0), moe(2, 2, 32, (2, 2), 1.0, 16)),
    layer(mixer(8, 16, 8, 16, 128, 50, 8, 7000.0, 0.5), moe(5, 2, 16, None, 0.7, 8)),
    layer(mixer(5, 8, 16, 24, 24, 0, 16, 1.0e6, 0.4), None),
    layer(mixer(16, 8, 8, 8, 32, 100, 8, 300.0), moe(9, 3, 8, (3, 1), 0.5, 24)),
], bigram=(1, 1, 1), scale=1.0, eps=3e-6)

# sizes that are multiples of nothing (float32 only)
ODD = model(50, 199, [
    layer(mixer(3, 10, 6, 7, 13, 5, 4, 777.0), moe(5, 2, 11, None, 1.3, 9)),
    layer(mixer(2, 5, 2, 9, 21, 12, 2, 10.0), moe(6, 4, 3, (2, 2), 1.0, None)),
], bigram=(31, 1000003, 999983), scale=0.5)

ONLY_ATTENTION = model(64, 199, [layer(mixer(6, 16, 16, 8, 64, 20, 16), None)], bigram=(50, 3, 5))
ONLY_MOE = model(64, 199, [layer(mixer(2, 8, 8, 8, 16, 9, 8), moe(8, 3, 16, (4, 2), 2.0, 24))], bigram=(11, 2, 9))
# no pair table: the token rows times the scale alone
NO_PAIRS = model(64, 150, [layer(mixer(2, 16, 8, 16, 32, 12, 8), moe(3, 2, 8))], bigram=None, scale=2.0)

CONFIGS = {"A": (MIX_A, 16), "B": (MIX_B, 8), "odd": (ODD, 4), "attention": (ONLY_ATTENTION, 4), "moe": (ONLY_MOE, 16),
           "no_pairs": (NO_PAIRS, 8)}


def every_expert(cfg):
    """The same model with every expert chosen by every token (and every group kept): its routing cannot
    flip where two scores are close, so a bfloat16 engine and the plain model choose alike."""
    out = copy.deepcopy(cfg)
    for l in out["layers"]:
        if l["mlp"]:
            r = l["mlp"]["router"]
            r["top"] = r["experts"]
            if r.get("groups"):
                r["groups"]["keep"] = r["groups"]["count"]
    return out


def random_config(seed, multiple=8):
    """A configuration drawn at random: width, vocabulary, bigram constants, two to four layers that each draw
    their own head count and sizes, latent, window, rotated dims and feed-forward."""
    import random
    rng = random.Random(seed)
    m = multiple
    width = rng.choice([64, 96, 128, 192, 256])
    layers = []
    for _ in range(rng.randrange(2, 5)):
        heads = rng.choice([1, 2, 3, 4, 6, 8, 12, 16, 24])
        dim = m * rng.randrange(1, 9)
        rot_dim = rng.choice([0, 8, 16, 32, 64])
        vdim = m * rng.randrange(1, 12)
        kv_rank = rng.choice([16, 24, 32, 48, 64, 80, 96, 128, 200, 256])
        window = rng.choice([0, 1, 2, 5, 16, 31, 64, 100, 5000])
        rot_dims = rng.choice([rot_dim, max(2, rot_dim // 2)]) if rot_dim else None
        a = mixer(heads, dim, rot_dim, vdim, kv_rank, window, rot_dims, rng.choice([100.0, 10000.0, 250000.0]))
        kind = rng.choice(["moe", "moe", "moe", "none"])
        mlp = None
        if kind == "moe":
            count = rng.choice([1, 1, 2, 3, 4])
            per = rng.randrange(1, 5)
            e = count * per
            keep = rng.randrange(1, count + 1)
            top = rng.randrange(1, keep * per + 1)
            mlp = moe(e, top, m * rng.randrange(1, 12), (count, keep) if count > 1 or rng.random() < 0.3 else None,
                      rng.choice([1.0, 2.0, 0.5]), rng.choice([None, m * rng.randrange(1, 12)]))
        layers.append(layer(a, mlp))
    return model(width, rng.randrange(90, 700), layers,
                 bigram=(rng.randrange(1, 2000), rng.randrange(1, 100), rng.randrange(1, 100)),
                 scale=rng.choice([1.0, 4.0, 11.0]), eps=rng.choice([1e-5, 1e-6, 1e-4]))


def random_weights(cfg, seed=0, sharpen=3.0):
    """{name: tensor} (float32).  `sharpen`: the gain of the projections that make scores and gates (3: far from
    uniform, a misplaced key or a lost sink moves the logits; 1: tame, so that bfloat16 rounding is not amplified)."""
    lively = 2.0 if sharpen > 1.0 else 1.0
    rng = np.random.default_rng(seed)
    W, V, out = cfg["width"], cfg["vocab"], {}

    def mat(name, rows, cols, gain=1.0):
        out[name] = rng.standard_normal((rows, cols)) * gain / np.sqrt(cols)

    def vec(name, n, mean=0.0, std=0.1):
        out[name] = mean + std * rng.standard_normal(n)

    mat("embed", V, W, gain=np.sqrt(W) / max(cfg["embedding"].get("scale", 1.0), 1.0))
    if cfg["embedding"].get("bigram"):
        out["bigram"] = 0.7 * rng.standard_normal((cfg["embedding"]["bigram"]["buckets"] + 1, W))
    for i, l in enumerate(cfg["layers"]):
        p, a = f"l{i}.", l["mixer"]
        H, D, R, Vd, C = a["heads"], a["dim"], a["rot_dim"], a["vdim"], a["kv_rank"]
        vec(p + "norm1", W, 1.0, 0.2)
        mat(p + "mix.q", H * (D + R), W, gain=sharpen)
        mat(p + "mix.dkv", C + R, W, gain=sharpen)
        vec(p + "mix.dkv.norm", C, 1.0, 0.2)
        mat(p + "mix.uk", H * D, C, gain=1.0)
        mat(p + "mix.uv", H * Vd, C)
        vec(p + "mix.sink", H, 0.0, 1.5 if sharpen > 1.0 else 0.5)
        mat(p + "mix.g", H * Vd, W, gain=lively)
        mat(p + "mix.o", W, H * Vd)
        mlp = l["mlp"]
        if mlp is not None:
            vec(p + "norm2", W, 1.0, 0.2)
            F = mlp["expert"]["ff"]
            for e in range(mlp["router"]["experts"]):
                mat(p + f"mlp.e{e}.up", F, W, gain=lively)
                mat(p + f"mlp.e{e}.down", W, F)
            mat(p + "mlp.router", mlp["router"]["experts"], W, gain=2.0 * lively)
            if mlp.get("shared"):
                mat(p + "mlp.shared.up", mlp["shared"]["ff"], W, gain=lively)
                mat(p + "mlp.shared.down", W, mlp["shared"]["ff"])
    vec("final.norm", W, 1.0, 0.2)
    mat("head", V, W, gain=lively)
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
