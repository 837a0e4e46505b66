"""A plain, slow Vevapel: every mechanism of the design as one small function, written from its
equations with torch on the CPU (float64 unless told otherwise).  It shares no code with the
engine: it reads config.json's own keys and the checkpoint's tensor names, keeps whole sequences
(no cache, no pages, no state slots) and runs one request at a time.

Notation: x [T, W] is the residual stream; weights are [out, in] and applied as h @ W.T; LN is a
layer norm with weight and bias; a layer is x <- x + m LN1b(mixer(LN1(x))), then
x <- x + m LN2b(ffn(LN2(x))), m a constant of the model.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


# --------------------------------------------------------------------------- norms
def layer_norm(x, w, b, eps):
    """(x - mean) / sqrt(mean squared deviation + eps) * w + b over the last axis."""
    mu = x.mean(dim=-1, keepdim=True)
    d = x - mu
    return d / torch.sqrt((d * d).mean(dim=-1, keepdim=True) + eps) * w + b


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


# ------------------------------------------------------------------------ rotation
def rotate_half(x, positions, dims: int, base: float):
    """x [T, ..., D]: of the last axis the first `dims` rotate, element i paired with i + dims/2, by the
    angle p * base^(-2i/dims); the rest passes."""
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    a = positions.to(torch.float64)[:, None] * f[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    cos, sin = torch.cos(a).reshape(shape).to(x.dtype), torch.sin(a).reshape(shape).to(x.dtype)
    u, v = x[..., :half], x[..., half:dims]
    out = x.clone()
    out[..., :half] = u * cos - v * sin
    out[..., half:dims] = v * cos + u * sin
    return out


# --------------------------------------------------------------------------- masks
def causal(positions):
    """allowed[i, j]: the query at positions[i] sees the key at positions[j] if j <= i."""
    return positions[None, :] <= positions[:, None]


def same_chunk(positions, size: int):
    """Causal, and only inside the query's own run of `size` positions (runs begin at multiples of `size`)."""
    i, j = positions[:, None], positions[None, :]
    return (j <= i) & (torch.div(i, size, rounding_mode="floor") == torch.div(j, size, rounding_mode="floor"))


def softmax_attend(q, k, v, allowed, scale):
    """q [T, H, D], k [T, H, D], v [T, H, V] (key/value heads already matched to query heads) -> [T, H, V]."""
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    s = s.masked_fill(~allowed[None], float("-inf"))
    p = torch.softmax(s, dim=-1)
    return torch.einsum("hij,jhv->ihv", p, v)


def query_temperature(positions, coef: float, every: int):
    """1 + coef ln(floor((p + 1) / every) + 1), one factor per position."""
    steps = torch.div(positions + 1, every, rounding_mode="floor").to(torch.float64)
    return 1.0 + coef * torch.log(steps + 1.0)


# ----------------------------------------------------------- mixer: gated attention
def attention(h, w, m, eps, positions):
    """Grouped-query softmax attention without rotation: biases on q, k, v and the output; one RMS norm over
    a token's WHOLE query projection (and key projection) with a weight per row; queries scaled by a factor
    that grows with the logarithm of the position; a sigmoid gate per head."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit_rms(h @ w["q"].T + w["q.b"], eps) * w["q.norm"]
    k = unit_rms(h @ w["k"].T + w["k.b"], eps) * w["k.norm"]
    v = h @ w["v"].T + w["v.b"]
    t = m.get("q_temp")
    if t:
        q = q * query_temperature(positions, t["coef"], t["every"]).to(q.dtype)[:, None]
    q, k, v = q.reshape(T, H, D), k.reshape(T, G, D), v.reshape(T, G, V)
    k, v = k.repeat_interleave(H // G, dim=1), v.repeat_interleave(H // G, dim=1)
    o = softmax_attend(q, k, v, causal(positions), m["scale"])
    gate = torch.sigmoid(h @ w["g"].T)                      # [T, H]
    o = o * gate[:, :, None]
    return o.reshape(T, H * V) @ w["o"].T + w["o.b"]


# ----------------------------------------------------- mixer: differential attention
def diff_lambda(w, diff: float):
    return torch.exp((w["lq1"] * w["lk1"]).sum()) - torch.exp((w["lq2"] * w["lk2"]).sum()) + diff


def attention_2(h, w, m, eps, positions):
    """Two softmax maps per head over the same values, the second subtracted lambda times; rotation on part of
    every map's dims; keys visible only inside the query's chunk; the head's result divided by its root mean
    square and multiplied by 1 - diff; a sigmoid gate per element."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T + w["q.b"]).reshape(T, H, 2, D)
    k = (h @ w["k"].T + w["k.b"]).reshape(T, G, 2, D)
    v = (h @ w["v"].T + w["v.b"]).reshape(T, G, V)
    rot = m.get("rot")
    if rot and rot.get("dims"):
        q = rotate_half(q, positions, rot["dims"], rot["base"])
        k = rotate_half(k, positions, rot["dims"], rot["base"])
    k, v = k.repeat_interleave(H // G, dim=1), v.repeat_interleave(H // G, dim=1)
    mask = m.get("mask")
    allowed = same_chunk(positions, mask["size"]) if mask else causal(positions)
    a1 = softmax_attend(q[:, :, 0], k[:, :, 0], v, allowed, m["scale"])
    a2 = softmax_attend(q[:, :, 1], k[:, :, 1], v, allowed, m["scale"])
    o = a1 - diff_lambda(w, m["diff"]) * a2
    o = unit_rms(o, eps) * (1.0 - m["diff"])
    o = o.reshape(T, H * V) * torch.sigmoid(h @ w["g"].T)
    return o @ w["o"].T


# -------------------------------------------------------------- mixer: the delta rule
def short_conv(x, taps_w):
    """x [T, C], taps_w [C, taps]: y[t, c] = sum_j taps_w[c, j] x[t - (taps - 1) + j, c], inputs ahead of the sequence count as zero."""
    T, taps = x.shape[0], taps_w.shape[1]
    pad = torch.cat([torch.zeros((taps - 1, x.shape[1]), dtype=x.dtype), x], dim=0)
    y = torch.zeros_like(x)
    for j in range(taps):
        y = y + pad[j:j + T] * taps_w[:, j]
    return y


def unit_vector(x):
    return x / torch.sqrt((x * x).sum(dim=-1, keepdim=True) + 1e-6)


def delta_scan(q, k, v, beta, g):
    """q, k [T, H, D], v [T, H, V], beta, g [T, H].  Per head, token by token:
    S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q."""
    T, H, D = q.shape
    V = v.shape[-1]
    S = torch.zeros((H, D, V), dtype=q.dtype)
    out = torch.zeros((T, H, V), dtype=q.dtype)
    for t in range(T):
        S = S * g[t][:, None, None]
        u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
        S = S + torch.einsum("hd,hv->hdv", k[t], u)
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out


def delta(h, w, m, eps, positions=None):
    """The gated delta rule with one decay per head."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ w["q"].T, w["q.conv"])).reshape(T, G, D)
    k = silu(short_conv(h @ w["k"].T, w["k.conv"])).reshape(T, G, D)
    v = silu(short_conv(h @ w["v"].T, w["v.conv"])).reshape(T, H, V)
    q = unit_vector(q) * D ** -0.5
    k = unit_vector(k)
    q, k = q.repeat_interleave(H // G, dim=1), k.repeat_interleave(H // G, dim=1)
    beta = torch.sigmoid(h @ w["b"].T)
    g = torch.exp(-torch.exp(w["A_log"]) * torch.nn.functional.softplus(h @ w["a"].T + w["dt_bias"]))
    o = delta_scan(q, k, v, beta, g)
    o = unit_rms(o, eps) * w["norm"]
    o = o.reshape(T, H * V) * silu(h @ w["g"].T)
    return o @ w["o"].T


MIXERS = {"attention": attention, "attention_2": attention_2, "delta": delta}


# ------------------------------------------------------------------------- experts
def route(h, w_router, b_router, top: int):
    """The `top` largest logits of each token and the softmax over just those: (ids [T, top], weights [T, top])."""
    z = h @ w_router.T + b_router
    val, ids = torch.topk(z, top, dim=-1)
    return ids, torch.softmax(val, dim=-1)


def expert(h, w, prefix):
    return (silu(h @ w[prefix + ".gate"].T) * (h @ w[prefix + ".up"].T)) @ w[prefix + ".down"].T


def moe(h, w, mlp):
    ids, wts = route(h, w["router"], w["router.b"], mlp["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(ids.shape[1]):
            out[t] = out[t] + wts[t, j] * expert(h[t:t + 1], w, f"e{int(ids[t, j])}")[0]
    return out


# --------------------------------------------------------------------------- model
def sub(weights: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    n = len(prefix)
    return {k[n:]: v for k, v in weights.items() if k.startswith(prefix)}


def run_order(cfg):
    """The layers in the order they run: (layer, pass number or None, first of its pass)."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None, False) for i in range(n)]
    order = [(i, None, False) for i in range(loop["start"])]
    for t in range(loop["times"]):
        order += [(i, t, i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return order + [(i, None, False) for i in range(loop["stop"], n)]


def forward(cfg, weights, tokens, dtype=torch.float64, trace: Optional[List[torch.Tensor]] = None, round_inputs=None):
    """Logits [T, vocab] of one sequence; `trace` collects the residual stream after every layer run.
    round_inputs (a torch dtype): every sublayer's normed input is rounded to it and back, the one rounding that
    any engine with products in that type must make; what it does to the logits says how far two correct
    implementations in that type may lie apart."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps, m = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    positions = torch.arange(len(tokens))
    x0 = w["embed"][torch.tensor(list(tokens), dtype=torch.long)] * cfg.get("embedding", {}).get("scale", 1.0)
    x = x0
    for i, t, first in run_order(cfg):
        if first:
            x = torch.cat([x, x0], dim=-1) @ w["loop.in"].T + w["loop.step"][t]
        layer, p = cfg["layers"][i], f"l{i}."
        ln = lambda name, y: layer_norm(y, w[p + name], w[p + name + ".b"], eps)
        cut = (lambda h: h.to(round_inputs).to(dtype)) if round_inputs is not None else (lambda h: h)
        y = MIXERS[layer["type"]](cut(ln("norm1", x)), sub(w, p + "mix."), layer["mixer"], eps, positions)
        x = x + m * ln("norm1b", y)
        if layer.get("mlp"):
            y = moe(cut(ln("norm2", x)), sub(w, p + "mlp."), layer["mlp"])
            x = x + m * ln("norm2b", y)
        if trace is not None:
            trace.append(x.clone())
    x = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
    return x @ w["embed"].T
