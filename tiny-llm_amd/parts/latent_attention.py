"""Causal attention whose cache holds one latent vector per token instead of keys and values.

Per token (h is the mixer's input, [out, in] weights applied as W h):
    c_q = w_dqn * unit_rms(W_dq h)                 q = W_uq c_q, per head [dim unrotated | rot_dim rotated]
    [c_raw | kr_raw] = W_dkv h                     c = w_dkvn * unit_rms(c_raw), kr = rotate(kr_raw)
    head n:  k_n = [W_uk,n c | kr],  v_n = W_uv,n c
    score = (q_unrotated . W_uk,n c + rotate(q_rotated) . kr) * scale, softmax over positions j <= i
    out = W_o concat_n( sigmoid(W_g h)_n * sum_j p_j v_j )
Only c and kr are cached (pages [block, kv_rank] and [block, rot_dim]).  A layer built with
`shares_cache=True` has no W_dkv: the plan lets it read the cache of an earlier layer, with its own
W_uk, W_uv and queries.

Options, each by itself:
    q_rank = 0        no query latent: q = W_q h directly (tensor `q`)
    window = w        position i sees j with 0 <= i - j < w; the cache gives pages back behind the window
    sink              a learned number per head (tensor `sink`) whose exponential joins the softmax's
                      denominator; it has no key and no value and is not scaled
    gate              "head": one sigmoid(W_g h) per token and head (W_g [heads, W]); "element": one per
                      element of the concatenated heads (W_g [heads * vdim, W]); None
    position.pairing  "half" (i, i + dims/2) or "interleaved" (2i, 2i + 1)

The up projections never touch the cache: q' = W_uk,n^T q_unrotated is formed per query
([T, heads, kv_rank], float32), the kernel scores [q' | q_rotated] against [c | kr] and returns
sum_j p_j c_j, and W_uv,n is applied to that.  The cache is read once per head as it lies, whatever
the cut of the prompt; nothing of the context is projected again when a portion arrives.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .base import CacheSpec, CacheTensor, LayerCache, Mixer, POSITION_ENCODINGS, WeightSpec, register_mixer
from .norm import LazyNorm


def _pad8(n: int) -> int:
    return -(-n // 8) * 8


class LatentAttention(Mixer):
    graph_safe = True
    accepts_lazy_norm = True        # a pre-norm block's norm rides in the one product that reads h

    def __init__(self, prefix, dtype, device, *, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int,
                 value_dim: int, q_rank: int, kv_rank: int, scale: float, eps: float, position: dict = None,
                 shares_cache: bool = False, gated: bool = True, names: Dict[str, str] = None, window: int = 0,
                 sink: bool = False, gate: str = "default"):
        """head_dim: unrotated query/key dims per head; rot_dim: rotated dims behind them (the position
        encoding rotates its first `rotary_dim`); scale: the factor of the scores, as given; `gated` is the
        older spelling of gate="head" / gate=None."""
        super().__init__(prefix, dtype, device)
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.head_dim, self.rot_dim, self.value_dim = int(head_dim), int(rot_dim), int(value_dim)
        self.q_rank, self.kv_rank = int(q_rank), int(kv_rank)
        self.scale, self.eps = float(scale), float(eps)
        self.shares_cache = bool(shares_cache)
        self.gate = ("head" if gated else None) if gate == "default" else gate
        if self.gate not in (None, "head", "element"):
            raise ValueError(f"{prefix}: gate is None, 'head' or 'element', got {gate!r}")
        self.gated = self.gate is not None
        self.window, self.sink = int(window or 0), bool(sink)
        if min(self.num_heads, self.head_dim, self.value_dim, self.kv_rank) <= 0 or self.q_rank < 0 or self.window < 0:
            raise ValueError(f"{prefix}: heads, head sizes and ranks must be positive, q_rank and window not negative")
        if self.window and self.shares_cache:
            raise ValueError(f"{prefix}: a layer with a window keeps a cache of its own")
        ops.check_latent_sizes(self.kv_rank, self.rot_dim)
        for n, what in ((self.hidden_size, "hidden_size"), (self.q_rank or 8, "q_rank"), (self.kv_rank, "kv_rank"),
                        (self.head_dim, "head_dim"), (self.head_dim + self.rot_dim, "head_dim + rot_dim"),
                        (self.num_heads * self.value_dim, "heads * value_dim"), (self.value_dim, "value_dim")):
            ops.check_linear_sizes(dtype, n, f"{prefix}: {what}")
        pos = dict(position or {"kind": "none"})
        kind = pos.pop("kind")
        self.position = POSITION_ENCODINGS.get(kind)(f"{prefix}.position", dtype, device, **pos)
        tables = self.position.rotary_tables()
        self.pairing = getattr(self.position, "pairing", "half")
        if (tables is None) != (self.rot_dim == 0) or self.pairing not in ops.ROPE_PAIRINGS:
            raise ValueError(f"{prefix}: rot_dim dims need a rotary encoding, paired {' or '.join(ops.ROPE_PAIRINGS)}")
        self.rdims = tables[2] if tables is not None else 0
        if self.rdims > self.rot_dim:
            raise ValueError(f"{prefix}: the encoding rotates {self.rdims} dims, the head has {self.rot_dim} for it")
        n = {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "q": "q", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk",
             "uv": "uv", "g": "g", "o": "o", "sink": "sink"}
        n.update(names or {})
        self.names = {k: f"{prefix}.{v}" for k, v in n.items()}
        # columns of the one product that reads h: [query latent, or the queries themselves | latent and key
        # part | gate], each starting at a multiple of 8 (the rows between are zero)
        self.q_width = self.num_heads * (self.head_dim + self.rot_dim)
        self.gate_width = {None: 0, "head": self.num_heads, "element": self.num_heads * self.value_dim}[self.gate]
        self.q_off = 0
        self.kv_off = _pad8(self.q_rank or self.q_width)
        self.g_off = self.kv_off + (0 if self.shares_cache else _pad8(self.kv_rank + self.rot_dim))
        self.down_width = self.g_off + _pad8(self.gate_width)
        self.w_down = self.w_uq = self.w_uk_t = self.w_uv = self.w_o = self.w_uk_few = self.w_uv_few = None
        self.w_dq_norm = self.w_dkv_norm = self.sinks = None

    # ---------------------------------------------------------------- declarations
    def weights(self) -> List[WeightSpec]:
        n, W, H = self.names, self.hidden_size, self.num_heads
        if self.q_rank:
            out = [WeightSpec(n["dq"], (self.q_rank, W)),
                   WeightSpec(n["dq_norm"], (self.q_rank,), role="vector", init="ones"),
                   WeightSpec(n["uq"], (self.q_width, self.q_rank))]
        else:
            out = [WeightSpec(n["q"], (self.q_width, W))]
        if not self.shares_cache:
            out += [WeightSpec(n["dkv"], (self.kv_rank + self.rot_dim, W)),
                    WeightSpec(n["dkv_norm"], (self.kv_rank,), role="vector", init="ones")]
        out += [WeightSpec(n["uk"], (H * self.head_dim, self.kv_rank)),
                WeightSpec(n["uv"], (H * self.value_dim, self.kv_rank))]
        if self.sink:
            out.append(WeightSpec(n["sink"], (H,), role="vector", init="normal"))
        if self.gated:
            out.append(WeightSpec(n["g"], (self.gate_width, W)))
        out.append(WeightSpec(n["o"], (W, H * self.value_dim)))
        return out

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        n, H = self.names, self.num_heads
        first = tensors[n["dq"] if self.q_rank else n["q"]]
        down = torch.zeros((self.down_width, self.hidden_size), dtype=self.dtype, device=first.device)
        down[:first.shape[0]] = first
        if not self.shares_cache:
            down[self.kv_off:self.kv_off + self.kv_rank + self.rot_dim] = tensors[n["dkv"]]
            self.w_dkv_norm = tensors[n["dkv_norm"]].to(torch.float32).contiguous()
        if self.gated:
            down[self.g_off:self.g_off + self.gate_width] = tensors[n["g"]]
        self.w_down = down
        if self.q_rank:
            self.w_dq_norm = tensors[n["dq_norm"]].to(torch.float32).contiguous()
            self.w_uq = tensors[n["uq"]].contiguous()
        if self.sink:
            self.sinks = tensors[n["sink"]].to(torch.float32).contiguous()
        # per head the transpose of W_uk: q' = W_uk^T q is a product with [kv_rank, head_dim] weights
        uk = tensors[n["uk"]].view(H, self.head_dim, self.kv_rank)
        self.w_uk_t = uk.transpose(1, 2).contiguous()
        self.w_uv = tensors[n["uv"]].contiguous()
        # the same two as [heads, inner, cols], for the one-launch products of steps with few rows
        self.w_uk_few = ops.head_product_weights(uk)
        self.w_uv_few = ops.head_product_weights(self.w_uv.view(H, self.value_dim, self.kv_rank).transpose(1, 2))
        # for steps of few rows the value products are rows against the weights of each row's own head: row t * H + n
        # takes head n (the table the per-row kernel of the experts looks its weights up in)
        self.head_of_row = (torch.arange(ops.HEAD_PRODUCT_ROWS * H, dtype=torch.int32, device=self.w_uv.device) % H
                            ).reshape(-1, 1).contiguous()
        self.w_o = tensors[n["o"]].contiguous()

    def cache_spec(self) -> CacheSpec:
        tensors = [CacheTensor("latent", (self.kv_rank,), 0)]
        if self.rot_dim:
            tensors.append(CacheTensor("rope_key", (self.rot_dim,), 0))
        return CacheSpec(tuple(tensors), "window" if self.window else "full", self.window)

    # --------------------------------------------------------------------- compute
    def forward(self, h, ctx, cache: LayerCache, state, residual):
        if cache.write == self.shares_cache:
            raise ValueError(f"{self.prefix}: a layer with a down projection of its own writes its cache, "
                             "one without reads another layer's")
        lazy = h if isinstance(h, LazyNorm) else None
        T, dev, H = (lazy.num_rows, lazy.x.device, self.num_heads) if lazy is not None else (h.shape[0], h.device, self.num_heads)
        R, D, V, KR = self.rot_dim, self.head_dim, self.value_dim, self.kv_rank
        tables = self.position.rotary_tables()
        cos, sin = (tables[0], tables[1]) if tables is not None else (None, None)
        latent, rope = cache.tensors["latent"], cache.tensors.get("rope_key")
        down = ops.scratch("latent_down", (T, self.down_width), self.dtype, dev)
        if lazy is not None:
            lazy.linear(self.w_down, down)
        else:
            ops.linear(h, self.w_down, down)
        kv = () if self.shares_cache else (self.kv_off, KR, R, self.rdims, self.w_dkv_norm, ctx.positions, cos, sin,
                                           ctx.slot_mappings[cache.group], latent, rope, self.pairing)
        if self.q_rank:
            cq = ops.scratch("latent_cq", (T, self.q_rank), self.dtype, dev)
            ops.latent_prepare(down, self.q_off, self.q_rank, self.w_dq_norm, self.eps, cq, *kv)
            q = ops.scratch("latent_q", (T, self.q_width), self.dtype, dev)
            ops.linear(cq, self.w_uq, q)
        else:
            if kv:
                ops.latent_prepare(down, 0, 0, None, self.eps, None, *kv)
            q = down[:, :self.q_width]                   # the queries came out of the one product
        # [W_uk^T q_unrotated | rotate(q_rotated)] per head, float32
        qa = ops.scratch("latent_qa", (T, H, KR + R), torch.float32, dev)
        q3, qa2 = q.unflatten(1, (H, D + R)), qa.view(T, H * (KR + R))
        few = T <= ops.HEAD_PRODUCT_ROWS and max(D, KR) <= ops.HEAD_PRODUCT_INNER
        many = self.dtype == torch.bfloat16 and not few and q.stride(0) % 8 == 0     # one launch on the matrix cores
        if few:
            ops.head_products(q3[:, :, :D], self.w_uk_few, qa[:, :, :KR])
        elif many:
            ops.head_gemm(q3[:, :, :D], self.w_uk_t, qa[:, :, :KR])
        else:
            for n in range(H):
                ops.linear(q3[:, n, :D], self.w_uk_t[n], qa2[:, n * (KR + R):n * (KR + R) + KR])
        if R:
            ops.rotate_into(q, H, D + R, D, R, self.rdims, ctx.positions, cos, sin, qa, KR, self.pairing)
        mix = ops.scratch("latent_mix", (T, H, KR), self.dtype, dev)
        gate = down[:, self.g_off:self.g_off + H] if self.gate == "head" else None
        extra = dict(window=self.window, sinks=self.sinks)
        if ops.latent_flash_supported(self.dtype, KR, R):
            # bfloat16: on the matrix cores, 16 heads of a token (or 16 / heads tokens) a tile
            decode = ctx.max_q_len == 1 and T == ctx.num_requests
            tpt = 16 // min(H, 16)
            if not decode and T >= ops.LATENT_PREFILL_ROWS:
                # many rows: four times the tokens a workgroup, which share every staged key tile
                ops.latent_prefill(qa, latent, rope, ctx.block_tables[cache.group], ctx.attention_tiles(4 * tpt),
                                   ctx.positions, mix, self.scale, gate, **extra)
                return self._project_heads(mix, down, residual, few, many)
            tiles = None if decode else ctx.attention_tiles(tpt)
            n_tiles = T if decode else tiles[0].numel()
            # the keys a tile walks at most: a window bounds them whatever the context
            span = min(ctx.max_seq_len, self.window + tpt + 14) if self.window else ctx.max_seq_len
            n_splits = ops.latent_key_splits(n_tiles * -(-H // 16), span)
            part = None
            if n_splits > 1:
                part = ops.scratch("attention_partials", (n_splits * T * H * (KR + 2),), torch.float32, dev)
            ops.latent_flash(qa, latent, rope, ctx.block_tables[cache.group], tiles, ctx.positions, mix, self.scale,
                             gate, n_splits, part, **extra)
        else:
            ops.latent_attention(qa, latent, rope, ctx.block_tables[cache.group], ctx.req_of_token, ctx.positions,
                                 mix, self.scale, gate, **extra)
        return self._project_heads(mix, down, residual, few, many)

    def _project_heads(self, mix, down, residual, few: bool, many: bool):
        """W_o concat_n(W_uv,n mix_n), with the per-head products as one launch where a kernel takes them, and the
        gate per element (its pre-activations lie in `down`) between the two."""
        T, H, KR = mix.shape
        V, dev = self.value_dim, mix.device
        o = ops.scratch("latent_heads", (T, H * V), self.dtype, dev)
        gate = down[:, self.g_off:self.g_off + H * V] if self.gate == "element" else None
        if few and KR >= 256:
            # a long inner size and few columns a head: a wave a group of four columns of one (token, head), its lanes
            # striding over the latent, fills the chip where a workgroup per 64 columns of a head leaves it idle
            ops.table_moe_up(mix.view(T * H, KR), self.w_uv.view(H, V, KR), None, self.head_of_row, o.view(T * H, V))
            if gate is not None:
                ops.gate_rows(o, gate, o)
        elif few:
            ops.head_products(mix, self.w_uv_few, o.view(T, H, V), gate)      # the gate rides in the product
        elif many:
            ops.head_gemm(mix, self.w_uv.view(H, V, KR), o.view(T, H, V), gate)
        else:
            for n in range(H):
                ops.linear(mix[:, n, :], self.w_uv[n * V:(n + 1) * V], o[:, n * V:(n + 1) * V])
            if gate is not None:
                ops.gate_rows(o, gate, o)
        if residual is None:
            return ops.linear(o, self.w_o, ops.scratch("sublayer_out", (T, self.hidden_size), torch.float32, dev))
        return ops.linear(o, self.w_o, residual, residual)


register_mixer("latent_attention", LatentAttention)
