"""Typed configuration of the Vevapel architecture, read from config.json keys.

config.json of this design is nested: `embedding.scale`; `layers` (the layers in order, each with `type`, which
mixer: `attention`, `delta` or `attention_2`; `mixer`, its sizes and constants; and `mlp`, a mixture of experts or
null for none); `loop` (`start`, `stop`, `times`: the layers from `start` up to but not including `stop` are run `times` times over on
the same weights, pass after pass; absent: every layer runs once); `norm.eps`; `residual_mult`; `vocab`; `width`.  Every size and constant
that can differ between models of the design comes from there; a layer has its own.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Sequence, Tuple, Union

from .llama import ConfigError

MIXERS = ("attention", "delta", "attention_2")
MLP_KINDS = ("moe",)
DEFAULT_MAX_POSITION = 131072       # the design has no limit of its own; the angle tables need one


@dataclass(frozen=True)
class GatedAttentionConfig:
    """`attention`: one score map, no rotation, a norm over the whole q and k projections, a gate per head."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    temp_coef: float        # query temperature 1 + coef ln(floor((p + 1) / every) + 1); every = 0: none
    temp_every: int


@dataclass(frozen=True)
class DiffAttentionConfig:
    """`attention_2`: two score maps per head, rotation on part of each map's dims, a chunked mask."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    chunk: int              # 0: every earlier position is seen
    rot_dims: int           # 0: no rotation
    rot_base: float


@dataclass(frozen=True)
class DeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int


@dataclass(frozen=True)
class MoeConfig:
    experts: int
    top: int
    ff: int


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class VevapelLayer:
    type: str
    mixer: Union[GatedAttentionConfig, DiffAttentionConfig, DeltaConfig]
    mlp: Optional[MoeConfig]


@dataclass(frozen=True)
class VevapelConfig:
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    residual_mult: float
    layers: Tuple[VevapelLayer, ...]
    loop: Optional[LoopConfig]
    max_position: int
    eos_token_ids: Tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], shapes: Optional[Mapping[str, Sequence[int]]] = None) -> "VevapelConfig":
        missing = [k for k in ("vocab", "width", "layers", "norm") if d.get(k) is None]
        if missing:
            raise ConfigError(f"config.json lacks required keys: {', '.join(missing)}")
        if not isinstance(d["layers"], (list, tuple)) or not d["layers"]:
            raise ConfigError("`layers` must list at least one layer")
        readers = {"attention": _attention, "attention_2": _attention_2, "delta": _delta}
        layers = []
        for i, raw in enumerate(d["layers"]):
            kind = raw.get("type")
            if kind not in MIXERS:
                raise ConfigError(f"layer {i}: mixer type {kind!r} is not built; known: {', '.join(MIXERS)}")
            layers.append(VevapelLayer(kind, readers[kind](i, raw.get("mixer") or {}), _mlp(i, raw.get("mlp"))))
        eps = float(_need("norm", d["norm"], "eps"))
        if not eps > 0:
            raise ConfigError("norm.eps must be positive")
        loop = None
        if d.get("loop"):
            lp = d["loop"]
            loop = LoopConfig(int(_need("loop", lp, "start")), int(_need("loop", lp, "stop")), int(_need("loop", lp, "times")))
            if not (0 <= loop.start < loop.stop <= len(layers)) or loop.times < 1:
                raise ConfigError(f"loop: layers {loop.start} .. {loop.stop - 1} run {loop.times} times: the run must "
                                  f"lie within the {len(layers)} layers, hold at least one and run at least once")
            if shapes is not None and "loop.step" in shapes and tuple(shapes["loop.step"])[0] != loop.times:
                raise ConfigError(f"loop.step has {tuple(shapes['loop.step'])[0]} rows, loop.times = {loop.times} are expected")
        eos = d.get("eos_token_id")
        eos = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else (eos,)))
        cfg = cls(vocab=int(d["vocab"]), width=int(d["width"]), norm_eps=eps,
                  embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)),
                  residual_mult=float(d.get("residual_mult", 1.0)), layers=tuple(layers), loop=loop,
                  max_position=int(d.get("max_position") or DEFAULT_MAX_POSITION), eos_token_ids=eos)
        if cfg.vocab <= 0 or cfg.width <= 0 or cfg.max_position <= 0:
            raise ConfigError("vocab, width and max_position must be positive")
        return cfg

    def run_order(self):
        """The layers in the order they run: (layer, pass number if the run begins a pass of the loop, else None)."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, None) for i in range(n)]
        lp = self.loop
        order = [(i, None) for i in range(lp.start)]
        for t in range(lp.times):
            order += [(i, t if i == lp.start else None) for i in range(lp.start, lp.stop)]
        return order + [(i, None) for i in range(lp.stop, n)]


def _need(where, m: Mapping[str, Any], key: str):
    if not isinstance(m, Mapping) or m.get(key) is None:
        raise ConfigError(f"layer {where}: `{key}` is missing")
    return m[key]


def _positive(where, m: Mapping[str, Any], key: str) -> int:
    v = int(_need(where, m, key))
    if v <= 0:
        raise ConfigError(f"layer {where}: `{key}` must be positive, got {v}")
    return v


def _heads(i: int, m: Mapping[str, Any]):
    heads, kv = _positive(i, m, "heads"), _positive(i, m, "kv_heads")
    if heads % kv:
        raise ConfigError(f"layer {i}: heads = {heads} must be a multiple of kv_heads = {kv}")
    return heads, kv, _positive(i, m, "dim"), _positive(i, m, "vdim")


def _attention(i: int, m: Mapping[str, Any]) -> GatedAttentionConfig:
    heads, kv, dim, vdim = _heads(i, m)
    t = m.get("q_temp") or {}
    coef, every = float(t.get("coef", 0.0)), int(t.get("every", 0)) if t else 0
    if t and every <= 0:
        raise ConfigError(f"layer {i}: q_temp.every must be positive, got {every}")
    return GatedAttentionConfig(heads, kv, dim, vdim, float(_need(i, m, "scale")), coef, every)


def _attention_2(i: int, m: Mapping[str, Any]) -> DiffAttentionConfig:
    heads, kv, dim, vdim = _heads(i, m)
    rot = m.get("rot") or {}
    rot_dims = int(rot.get("dims", 0)) if rot else 0
    if rot_dims % 2 or not (0 <= rot_dims <= dim):
        raise ConfigError(f"layer {i}: rot.dims = {rot_dims} must be even and within dim = {dim}")
    mask = m.get("mask") or {}
    chunk = int(mask.get("size", 0)) if mask else 0
    if chunk < 0:
        raise ConfigError(f"layer {i}: mask.size must be positive, got {chunk}")
    diff = float(_need(i, m, "diff"))
    return DiffAttentionConfig(heads, kv, dim, vdim, float(_need(i, m, "scale")), diff, chunk, rot_dims,
                               float(rot.get("base", 10000.0)) if rot_dims else 0.0)


def _delta(i: int, m: Mapping[str, Any]) -> DeltaConfig:
    heads, kv, dim, vdim = _heads(i, m)
    return DeltaConfig(heads, kv, dim, vdim, _positive(i, m, "conv"))


def _mlp(i: int, m: Optional[Mapping[str, Any]]) -> Optional[MoeConfig]:
    if m is None:
        return None
    if m.get("kind") not in MLP_KINDS:
        raise ConfigError(f"layer {i}: feed-forward kind {m.get('kind')!r} is not built; known: {', '.join(MLP_KINDS)}")
    r = _need(i, m, "router")
    experts, top = _positive(f"{i} (mlp.router)", r, "experts"), _positive(f"{i} (mlp.router)", r, "top")
    if top > experts:
        raise ConfigError(f"layer {i}: a token uses top = {top} of {experts} experts")
    return MoeConfig(experts, top, _positive(f"{i} (mlp.expert)", _need(i, m, "expert"), "ff"))
