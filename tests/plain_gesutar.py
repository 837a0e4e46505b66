"""A plain, slow Gesutar: every mechanism of the design as one small function, written from its
equations with torch on the CPU (float64 unless told otherwise).  It shares no code with the
engine: it reads config.json's own keys and the checkpoint's tensor names, keeps whole sequences
(no cache, no pages, no state slots) and runs one request at a time.

Notation: x [T, W] is the residual stream; weights are [out, in] and applied as h @ W.T; a layer is
x <- x + mixer(rms(x) * norm1), then x <- x + ffn(rms(x) * norm2).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch


# --------------------------------------------------------------------------- norm
def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w


# ---------------------------------------------------------------------- embedding
def bigram_rows(tokens, buckets: int, mul_prev: int, mul_cur: int):
    """Row of the bigram table for every token of one sequence: the hash of (previous token, token);
    the sequence's first token, which has no previous one, takes the row behind the buckets."""
    rows = [buckets]
    for a, b in zip(tokens[:-1], tokens[1:]):
        rows.append((int(a) * mul_prev + int(b) * mul_cur) % buckets)
    return torch.tensor(rows, dtype=torch.long)


def embed(tokens, w, e):
    """Token rows times a constant, plus the bigram rows (if the model has a bigram table)."""
    x = w["embed"][torch.tensor(list(tokens), dtype=torch.long)] * e.get("scale", 1.0)
    b = e.get("bigram")
    if b:
        x = x + w["bigram"][bigram_rows(list(tokens), b["buckets"], b["mul_prev"], b["mul_cur"])]
    return x


# ------------------------------------------------------------------------ rotation
def rotate_pairs(x, positions, dims: int, base: float):
    """x [T, ..., D]: of the last axis the first `dims` rotate, element 2i paired with 2i + 1, by the
    angle p * base^(-2i/dims); the rest passes."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    a = positions.to(torch.float64)[:, None] * f[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    cos, sin = torch.cos(a).reshape(shape).to(x.dtype), torch.sin(a).reshape(shape).to(x.dtype)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


# ---------------------------------------------------------------------- attention
def sink_softmax(s, allowed, sink):
    """p_j = exp(s_j) / (exp(sink) + sum_allowed exp(s_j)): the sink has no key and no value."""
    s = s.masked_fill(~allowed, float("-inf"))
    m = torch.maximum(s.max(dim=-1, keepdim=True).values, sink)
    e = torch.exp(s - m)
    return e / (torch.exp(sink - m) + e.sum(dim=-1, keepdim=True))


def visible(positions, window: Optional[int]):
    """allowed[i, j]: the query at positions[i] sees the key at positions[j]."""
    i, j = positions[:, None], positions[None, :]
    ok = j <= i
    if window:
        ok = ok & (i - j < window)
    return ok


def latent_attention(h, w, m, eps, positions):
    """h [T, W] -> [T, W].  Keys and values of every head come from one latent per token; the rotated
    part of the key is one vector per token that all heads share."""
    T = h.shape[0]
    H, D, R, V, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (h @ w["q"].T).reshape(T, H, D + R)
    down = h @ w["dkv"].T
    c = rms_norm(down[:, :C], w["dkv.norm"], eps)
    kr = down[:, C:C + R]
    rot = m.get("rot")
    q_rot = q[:, :, D:]
    if rot and R:
        q_rot = rotate_pairs(q_rot, positions, rot["dims"], rot["base"])
        kr = rotate_pairs(kr, positions, rot["dims"], rot["base"])
    k = (c @ w["uk"].T).reshape(T, H, D)
    v = (c @ w["uv"].T).reshape(T, H, V)
    allowed = visible(positions, (m.get("mask") or {}).get("size"))
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for n in range(H):
        s = (q[:, n, :D] @ k[:, n].T + q_rot[:, n] @ kr.T) * m["scale"]
        out[:, n] = sink_softmax(s, allowed, w["sink"][n]) @ v[:, n]
    out = out.reshape(T, H * V) * torch.sigmoid(h @ w["g"].T)
    return out @ w["o"].T


# -------------------------------------------------------------------- feed-forward
def relu2_unit(h, up, down):
    return torch.relu(h @ up.T) ** 2 @ down.T


def route(z, r):
    """Router logits z [T, E] -> (chosen experts [T, top], their weights [T, top])."""
    E, top = r["experts"], r["top"]
    s = torch.softmax(z, dim=-1)
    pick = s
    g = r.get("groups")
    if g and g["count"] > 1:
        per = E // g["count"]
        best = s.reshape(-1, g["count"], per).max(dim=-1).values
        kept = torch.zeros_like(best, dtype=torch.bool)
        kept.scatter_(1, best.topk(g["keep"], dim=-1).indices, True)
        pick = s.masked_fill(~kept.repeat_interleave(per, dim=1), -1.0)
    idx = pick.topk(top, dim=-1).indices
    wts = s.gather(1, idx)
    wts = wts / (wts.sum(dim=-1, keepdim=True) + 1e-20) * r.get("scale", 1.0)
    return idx, wts


def moe(h, w, m):
    """Routed experts (each token's chosen ones, weighted) plus the shared expert for every token."""
    r = m["router"]
    idx, wts = route((h @ w["router"].T), r)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(idx[t].tolist(), wts[t]):
            out[t] += a * relu2_unit(h[t:t + 1], w[f"e{e}.up"], w[f"e{e}.down"])[0]
    if m.get("shared"):
        out = out + relu2_unit(h, w["shared.up"], w["shared.down"])
    return out


# --------------------------------------------------------------------------- model
def sub(weights: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens, return_layers: bool = False):
    """Logits [T, vocab] of one whole sequence (and the residual stream behind every layer)."""
    positions = torch.arange(len(tokens))
    eps = cfg["norm"]["eps"]
    x = embed(tokens, weights, cfg.get("embedding") or {})
    streams: List[torch.Tensor] = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        if layer["type"] != "latent_attention":
            raise ValueError(f"layer {i}: unknown mixer {layer['type']!r}")
        h = rms_norm(x, weights[p + "norm1"], eps)
        x = x + latent_attention(h, sub(weights, p + "mix."), layer["mixer"], eps, positions)
        if layer.get("mlp") is not None:
            h = rms_norm(x, weights[p + "norm2"], eps)
            x = x + moe(h, sub(weights, p + "mlp."), layer["mlp"])
        streams.append(x)
    logits = rms_norm(x, weights["final.norm"], eps) @ weights["head"].T
    return (logits, torch.stack(streams)) if return_layers else logits
