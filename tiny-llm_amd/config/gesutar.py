"""Typed configuration of the Gesutar architecture, read from config.json keys.

config.json of this design is nested: `embedding` (a scale for the token rows and, under `bigram`, a
second table looked up by a hash of the token and the one before it: `buckets`, `mul_prev`, `mul_cur`),
`layers` (the layers in order, each with `type`, which mixer; `mixer`, its sizes; and `mlp`, a mixture of
experts or null for none), `norm.eps`, `vocab`, `width`.  Every size and constant that can differ between
models of the design comes from there; a layer has its own.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Sequence, Tuple

from .llama import ConfigError

MIXERS = ("latent_attention",)
MLP_KINDS = ("moe",)
DEFAULT_MAX_POSITION = 131072       # the design has no limit of its own; the angle tables need one


@dataclass(frozen=True)
class BigramConfig:
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass(frozen=True)
class WindowLatentConfig:
    heads: int
    dim: int            # unrotated query/key dims per head
    rot_dim: int        # rotated dims per head (the key's are one vector shared by all heads)
    vdim: int
    kv_rank: int
    scale: float
    window: int         # 0: every earlier position is seen
    rot_dims: int       # how many of rot_dim rotate
    rot_base: float


@dataclass(frozen=True)
class RoutedMoeConfig:
    experts: int
    top: int
    ff: int
    groups: int
    keep: int
    scale: float
    shared_ff: int      # 0: no shared expert


@dataclass(frozen=True)
class GesutarLayer:
    type: str
    mixer: WindowLatentConfig
    mlp: Optional[RoutedMoeConfig]


@dataclass(frozen=True)
class GesutarConfig:
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    bigram: Optional[BigramConfig]
    layers: Tuple[GesutarLayer, ...]
    max_position: int
    eos_token_ids: Tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], shapes: Optional[Mapping[str, Sequence[int]]] = None) -> "GesutarConfig":
        missing = [k for k in ("vocab", "width", "layers", "norm") if d.get(k) is None]
        if missing:
            raise ConfigError(f"config.json lacks required keys: {', '.join(missing)}")
        if not isinstance(d["layers"], (list, tuple)) or not d["layers"]:
            raise ConfigError("`layers` must list at least one layer")
        layers = []
        for i, raw in enumerate(d["layers"]):
            kind = raw.get("type")
            if kind not in MIXERS:
                raise ConfigError(f"layer {i}: mixer type {kind!r} is not built; known: {', '.join(MIXERS)}")
            layers.append(GesutarLayer(kind, _latent(i, raw.get("mixer") or {}), _mlp(i, raw.get("mlp"))))
        eps = float(_need("norm", d["norm"], "eps"))
        if not eps > 0:
            raise ConfigError("norm.eps must be positive")
        emb = d.get("embedding") or {}
        bigram = None
        if emb.get("bigram"):
            b = emb["bigram"]
            bigram = BigramConfig(_positive("embedding.bigram", b, "buckets"), int(_need("embedding.bigram", b, "mul_prev")),
                                  int(_need("embedding.bigram", b, "mul_cur")))
            if shapes is not None and "bigram" in shapes and tuple(shapes["bigram"])[0] != bigram.buckets + 1:
                raise ConfigError(f"the bigram table has {tuple(shapes['bigram'])[0]} rows, "
                                  f"embedding.bigram.buckets + 1 = {bigram.buckets + 1} are expected")
        eos = d.get("eos_token_id")
        eos = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else (eos,)))
        cfg = cls(vocab=int(d["vocab"]), width=int(d["width"]), norm_eps=eps,
                  embedding_scale=float(emb.get("scale", 1.0)), bigram=bigram, layers=tuple(layers),
                  max_position=int(d.get("max_position") or DEFAULT_MAX_POSITION), eos_token_ids=eos)
        if cfg.vocab <= 0 or cfg.width <= 0 or cfg.max_position <= 0:
            raise ConfigError("vocab, width and max_position must be positive")
        return cfg


def _need(where, m: Mapping[str, Any], key: str):
    if not isinstance(m, Mapping) or m.get(key) is None:
        raise ConfigError(f"layer {where}: `{key}` is missing")
    return m[key]


def _positive(where, m: Mapping[str, Any], key: str) -> int:
    v = int(_need(where, m, key))
    if v <= 0:
        raise ConfigError(f"layer {where}: `{key}` must be positive, got {v}")
    return v


def _latent(i: int, m: Mapping[str, Any]) -> WindowLatentConfig:
    rot_dim = int(m.get("rot_dim") or 0)
    rot = m.get("rot") or {}
    rot_dims = int(rot.get("dims") or rot_dim) if rot_dim else 0
    mask = m.get("mask") or {}
    cfg = WindowLatentConfig(heads=_positive(i, m, "heads"), dim=_positive(i, m, "dim"), rot_dim=rot_dim,
                             vdim=_positive(i, m, "vdim"), kv_rank=_positive(i, m, "kv_rank"),
                             scale=float(_need(i, m, "scale")), window=int(mask.get("size") or 0), rot_dims=rot_dims,
                             rot_base=float(_need(i, rot, "base")) if rot_dim else 0.0)
    if cfg.rot_dim < 0 or cfg.window < 0:
        raise ConfigError(f"layer {i}: rot_dim and mask.size must not be negative")
    if cfg.rot_dim and (cfg.rot_dims % 2 or not (0 < cfg.rot_dims <= cfg.rot_dim) or not cfg.rot_base > 0):
        raise ConfigError(f"layer {i}: rot.dims must be even and within rot_dim, rot.base positive")
    return cfg


def _mlp(i: int, m: Optional[Mapping[str, Any]]) -> Optional[RoutedMoeConfig]:
    if m is None:
        return None
    kind = m.get("kind", "moe")
    if kind not in MLP_KINDS:
        raise ConfigError(f"layer {i}: feed-forward kind {kind!r} is not built; known: {', '.join(MLP_KINDS)}")
    e, r = _need(i, m, "expert"), _need(i, m, "router")
    g = r.get("groups") or {}
    shared = m.get("shared") or {}
    cfg = RoutedMoeConfig(experts=_positive(i, r, "experts"), top=_positive(i, r, "top"), ff=_positive(i, e, "ff"),
                          groups=int(g.get("count") or 1), keep=int(g.get("keep") or g.get("count") or 1),
                          scale=float(r.get("scale", 1.0)), shared_ff=int(shared.get("ff") or 0))
    if cfg.top > cfg.experts:
        raise ConfigError(f"layer {i}: router.top {cfg.top} exceeds router.experts {cfg.experts}")
    if cfg.groups < 1 or cfg.experts % cfg.groups or not (0 < cfg.keep <= cfg.groups):
        raise ConfigError(f"layer {i}: router.groups.count must divide router.experts, and keep lie within it")
    if cfg.top > cfg.keep * (cfg.experts // cfg.groups):
        raise ConfigError(f"layer {i}: the {cfg.keep} kept groups hold fewer than router.top = {cfg.top} experts")
    if cfg.shared_ff < 0:
        raise ConfigError(f"layer {i}: mlp.shared.ff must be positive")
    return cfg
