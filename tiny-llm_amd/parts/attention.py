"""Grouped-query causal attention over the paged cache (the Llama mixer).

Per token: q, k, v = h Wq^T, h Wk^T, h Wv^T (tiny_llm/ops/cuda/gemm.cu:86-100,
head-major columns gemm.cu:119-123); q and k rotated by the token's position
(rope.cu:46-54); k (rotated) and v written to the cache (gemm.cu:400-407);
scores q.k * hd^-0.5 against the request's cached keys with a causal mask, online
softmax, weighted sum of values (flash_attention.cu:374-405); output projection
with the residual add folded in (gemm.cu:171-190, arithmetic.cu:13).

Q, K and V weights are concatenated on load into one [(nq + 2 nkv) * hd, H]
matrix: row concatenation leaves every dot product as it was.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .norm import LazyNorm
from .base import (CacheSpec, CacheTensor, LayerCache, Mixer, POSITION_ENCODINGS, WeightSpec, project_into_residual,
                   register_mixer)


class Attention(Mixer):
    graph_safe = True
    accepts_lazy_norm = True
    prepares_next_norm = True

    def __init__(self, prefix, dtype, device, *, hidden_size: int, num_heads: int, num_kv_heads: int,
                 head_dim: int, position: dict = None, window: int = 0, scale: float = None,
                 max_position: int = 0):
        super().__init__(prefix, dtype, device)
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        if self.num_kv_heads <= 0 or self.num_heads % self.num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        # sizes a kernel refuses are refused here, when the model is built, not at its first step
        ops.check_attention_sizes(dtype, self.num_heads, self.num_kv_heads, self.head_dim)
        ops.check_linear_sizes(dtype, self.hidden_size, f"{prefix}: hidden_size")
        ops.check_linear_sizes(dtype, self.num_heads * self.head_dim, f"{prefix}: num_heads * head_dim")
        self.window = int(window or 0)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        pos = dict(position or {"kind": "none"})
        kind = pos.pop("kind")
        self.position = POSITION_ENCODINGS.get(kind)(f"{prefix}.position", dtype, device, **pos)
        self.q_size = self.num_heads * self.head_dim
        self.kv_size = self.num_kv_heads * self.head_dim
        self.w_qkv: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None

    # ---------------------------------------------------------------- declarations
    def weights(self) -> List[WeightSpec]:
        p, H = self.prefix, self.hidden_size
        return [WeightSpec(f"{p}.q_proj.weight", (self.q_size, H)),
                WeightSpec(f"{p}.k_proj.weight", (self.kv_size, H)),
                WeightSpec(f"{p}.v_proj.weight", (self.kv_size, H)),
                WeightSpec(f"{p}.o_proj.weight", (H, self.q_size))]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        p = self.prefix
        self.w_qkv = torch.cat([tensors[f"{p}.q_proj.weight"], tensors[f"{p}.k_proj.weight"],
                                tensors[f"{p}.v_proj.weight"]], dim=0).contiguous()
        self.w_o = tensors[f"{p}.o_proj.weight"].contiguous()

    def cache_spec(self) -> CacheSpec:
        return CacheSpec.keys_and_values(self.num_kv_heads, self.head_dim, "window" if self.window else "full",
                                         self.window)

    # --------------------------------------------------------------------- compute
    def forward(self, h, ctx, cache: LayerCache, state, residual, next_norm=None):
        T = residual.shape[0]
        qkv = ops.scratch("qkv", (T, self.q_size + 2 * self.kv_size), self.dtype, residual.device)
        if isinstance(h, LazyNorm):
            h.linear(self.w_qkv, qkv)
        else:
            ops.linear(h, self.w_qkv, qkv)
        tables = self.position.rotary_tables()
        cos, sin, rot = tables if tables is not None else (None, None, 0)
        pairing = getattr(self.position, "pairing", "half")     # an encoding that says nothing pairs (i, i + rot/2)
        attn = ops.scratch("attention_out", (T, self.q_size), self.dtype, residual.device)
        q = qkv[:, :self.q_size]
        flash = ops.flash_attention_supported(self.dtype, self.num_heads, self.num_kv_heads, self.head_dim)
        # decode steps: rotation and cache write ride in the attention kernel
        fuse = flash and ctx.max_q_len == 1 and cache.write and rot == self.head_dim and pairing == "half"
        if not fuse:
            slots = ctx.slot_mappings[cache.group] if cache.write else None
            ops.rope_store(qkv, ctx.positions, cos, sin, slots, cache.k if cache.write else None,
                           cache.v if cache.write else None, self.num_heads, self.num_kv_heads, self.head_dim, rot,
                           pairing)
        self._attend(q, ctx, cache, attn, fused_rope=(cos, sin) if fuse else None)
        out, prepared = project_into_residual(attn, self.w_o, residual, next_norm)
        return out if next_norm is None else (out, prepared)

    def _attend(self, q, ctx, cache: LayerCache, attn, fused_rope=None, sink: bool = False):
        """attn <- attention of the step's query rows q [T, heads * head_dim] over the cache, by the kernel that
        takes this step's shape.  sink: one more term exp(0) in every softmax's denominator.  `self.window`: 0
        (every earlier key), n > 0 (the last n positions) or -n (the row's own run of n positions, runs counted
        from position 0: a chunked mask)."""
        T, device = q.shape[0], q.device
        group = self.num_heads // self.num_kv_heads
        flash = ops.flash_attention_supported(self.dtype, self.num_heads, self.num_kv_heads, self.head_dim)
        # the keys one row walks at most: a window bounds them whatever the context (the kernels begin at the
        # window's first key tile)
        span = min(ctx.max_seq_len, abs(self.window) + 63) if self.window else ctx.max_seq_len
        if flash and ctx.max_q_len > 1:
            # prompt portions: many query rows share each staged key tile
            waves = ops.prefill_tile_waves(T, self.num_heads, self.num_kv_heads)
            tiles = ctx.attention_tiles(waves * (16 // group))
            # a portion late in a long prompt: few query rows, many keys; the keys are shared out
            n_splits = ops.prefill_key_splits(T, span, self.num_heads, self.num_kv_heads, waves)
            scratch = None
            if n_splits > 1:
                scratch = ops.scratch("attention_partials", (n_splits * T * self.num_heads * (self.head_dim + 2),),
                                      torch.float32, device)
            ops.flash_prefill(q, cache.k, cache.v, ctx.block_tables[cache.group], tiles, ctx.positions, attn,
                              self.num_heads, self.num_kv_heads, self.head_dim, self.scale, self.window, waves,
                              n_splits, scratch, sink=sink)
        elif flash:
            # decoding: one token per request, its keys split over the waves of a workgroup (and over
            # workgroups when the context is long)
            # (no tile arrays when every request brings exactly one token: row i is request i)
            tiles = None if T == ctx.num_requests else ctx.attention_tiles(16 // group)
            n_splits, scratch = self._splits(span, T, device)
            ops.flash_attention(q, cache.k, cache.v, ctx.block_tables[cache.group], tiles, ctx.positions, attn,
                                self.num_heads, self.num_kv_heads, self.head_dim, self.scale, self.window,
                                n_splits, scratch, fused_rope=fused_rope, sink=sink)
        elif ops.attention_f32_supported(self.dtype, self.num_heads, self.num_kv_heads, self.head_dim) \
                and q.stride(0) % 4 == 0:
            # true float32 on the matrix cores; one fixed merge tree, so the same bits whatever the batch
            decode = ctx.max_q_len == 1 and T == ctx.num_requests
            tiles = None if decode else ctx.attention_tiles(16 // group)
            n_chunks = -(-ctx.max_seq_len // ops.F32_CHUNK_KEYS) if ctx.max_q_len == 1 else 1
            scratch = None
            if n_chunks > 1:
                scratch = ops.scratch("attention_partials", (n_chunks * T * self.num_heads * (self.head_dim + 2),),
                                      torch.float32, device)
            ops.attention_f32(q, cache.k, cache.v, ctx.block_tables[cache.group], tiles, ctx.positions, attn,
                              self.num_heads, self.num_kv_heads, self.head_dim, self.scale, self.window, n_chunks,
                              scratch, sink=sink)
        else:
            ops.paged_attention(q, cache.k, cache.v, ctx.block_tables[cache.group], ctx.req_of_token,
                                ctx.positions, attn, self.num_heads, self.num_kv_heads, self.head_dim,
                                self.scale, self.window, sink=sink)
        return attn

    def _splits(self, span: int, T: int, device):
        """How many workgroups share one query tile's keys (`ops.decode_key_splits`; `span`: the most keys a
        row walks), and the scratch for their partial results."""
        n_splits = ops.decode_key_splits(T, span, self.num_kv_heads, self.head_dim)
        if n_splits == 1:
            return 1, None
        return n_splits, ops.scratch("attention_partials", (n_splits * T * self.num_heads * (self.head_dim + 2),),
                                     torch.float32, device)


class NormedAttention(Attention):
    """Grouped-query attention over the paged cache whose queries and keys are prepared in float32 between
    their product and the attention kernel, each step an option of its own:

        q, k = W_q h (+ b_q), W_k h (+ b_k)             `bias`
        v    = k as projected (`values="keys"`, no W_v), or W_v h (`values="projected"`)
        q, k rotated on the first rotary_dim dims of every head (`position`, either pairing)
        q, k divided by their root mean square over the head (`qk_norm="unit"`, no weight, `eps`)
        p_j  = exp(s_j) / (1 + sum exp(s_j))            `sink`: a term of score 0 that carries no value
        head n's output times sigmoid(W_g h)_n          `head_gate`: one number per token and head
        result = out_scale * W_o concat_heads(...)

    `window` and `scale` as in `Attention`.  `names`: the tensors' names below the prefix (q, k, v, g, o;
    a bias is its matrix's name plus `bias_suffix`).  One product reads h for [q | k | (v) | g] and leaves
    float32; the gate and `out_scale` are applied to the attention's result in float32 before it is
    rounded for the output product.  With `residual=None` the result is returned by itself in float32."""
    graph_safe = True
    accepts_lazy_norm = False
    prepares_next_norm = False

    def __init__(self, prefix, dtype, device, *, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: dict = None, window: int = 0, scale: float = None, bias: bool = False,
                 values: str = "projected", qk_norm: str = None, eps: float = 1e-6, sink: bool = False,
                 head_gate: bool = False, out_scale: float = 1.0, names: Dict[str, str] = None,
                 bias_suffix: str = ".bias", max_position: int = 0):
        super().__init__(prefix, dtype, device, hidden_size=hidden_size, num_heads=num_heads,
                         num_kv_heads=num_kv_heads, head_dim=head_dim, position=position, window=window, scale=scale)
        if values not in ("projected", "keys"):
            raise ValueError(f"{prefix}: values are 'projected' or 'keys', got {values!r}")
        if qk_norm not in (None, "unit"):
            raise ValueError(f"{prefix}: qk_norm is None or 'unit', got {qk_norm!r}")
        if self.head_dim % 2:
            raise ValueError(f"{prefix}: head_dim {self.head_dim} must be even")
        if float(out_scale) != 1.0 and not head_gate:
            raise ValueError(f"{prefix}: out_scale rides in the head gate's kernel; without a gate it must be 1")
        self.bias, self.values_are_keys, self.unit_norm = bool(bias), values == "keys", qk_norm == "unit"
        self.eps, self.sink, self.head_gate, self.out_scale = float(eps), bool(sink), bool(head_gate), float(out_scale)
        n = {k: k for k in ("q", "k", "v", "g", "o")}
        n.update(names or {})
        self.names = {k: f"{prefix}.{v}" for k, v in n.items()}
        self.bias_suffix = bias_suffix
        # columns of the product that reads h: q heads, k heads, (v heads,) then the gates at a multiple of 8
        self.v_off = self.q_size + self.kv_size if not self.values_are_keys else -1
        used = self.q_size + self.kv_size * (1 if self.values_are_keys else 2)
        self.g_off = -(-used // 8) * 8
        self.in_width = self.g_off + (-(-self.num_heads // 8) * 8 if self.head_gate else 0)
        self.w_in = self.b_in = None

    def weights(self) -> List[WeightSpec]:
        n, H = self.names, self.hidden_size
        out = [WeightSpec(n["q"], (self.q_size, H)), WeightSpec(n["k"], (self.kv_size, H))]
        if self.bias:
            out += [WeightSpec(n["q"] + self.bias_suffix, (self.q_size,), role="vector", init="zeros"),
                    WeightSpec(n["k"] + self.bias_suffix, (self.kv_size,), role="vector", init="zeros")]
        if not self.values_are_keys:
            out.append(WeightSpec(n["v"], (self.kv_size, H)))
        if self.head_gate:
            out.append(WeightSpec(n["g"], (self.num_heads, H)))
        out.append(WeightSpec(n["o"], (H, self.q_size)))
        return out

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        n = self.names
        dev = tensors[n["q"]].device
        w = torch.zeros((self.in_width, self.hidden_size), dtype=self.dtype, device=dev)
        w[:self.q_size] = tensors[n["q"]]
        w[self.q_size:self.q_size + self.kv_size] = tensors[n["k"]]
        if not self.values_are_keys:
            w[self.v_off:self.v_off + self.kv_size] = tensors[n["v"]]
        if self.head_gate:
            w[self.g_off:self.g_off + self.num_heads] = tensors[n["g"]]
        self.w_in = w
        if self.bias:
            self.b_in = torch.cat([tensors[n["q"] + self.bias_suffix].to(torch.float32),
                                   tensors[n["k"] + self.bias_suffix].to(torch.float32)]).contiguous()
        self.w_o = tensors[n["o"]].contiguous()

    def forward(self, h, ctx, cache: LayerCache, state, residual):
        T, dev = h.shape[0], h.device
        p = ops.scratch("qk_product", (T, self.in_width), torch.float32, dev)
        ops.linear(h, self.w_in, p)
        tables = self.position.rotary_tables()
        cos, sin, rot = tables if tables is not None else (None, None, 0)
        pairing = getattr(self.position, "pairing", "half")
        q = ops.scratch("q_prepared", (T, self.q_size), self.dtype, dev)
        write = cache.write
        ops.qk_prepare(p, self.b_in, ctx.positions, cos, sin, ctx.slot_mappings[cache.group] if write else None, q,
                       cache.k if write else None, cache.v if write else None, self.num_heads, self.num_kv_heads,
                       self.head_dim, rot, pairing, self.unit_norm, self.eps, self.values_are_keys, self.v_off)
        attn = ops.scratch("attention_out", (T, self.q_size), self.dtype, dev)
        self._attend(q, ctx, cache, attn, sink=self.sink)
        if self.head_gate:
            ops.head_gate(attn, p[:, self.g_off:self.g_off + self.num_heads], attn, self.num_heads, self.head_dim,
                          self.out_scale)
        if residual is None:
            return ops.linear(attn, self.w_o, ops.scratch("sublayer_out", (T, self.hidden_size), torch.float32, dev))
        return ops.linear(attn, self.w_o, residual, residual)


class GatedAttention(Attention):
    """Grouped-query softmax attention over the paged cache whose head has `head_dim` query/key numbers and
    `value_dim` value numbers, with these options, each by itself:

        q, k, v = W_q h + b_q, W_k h + b_k, W_v h + b_v; the output product adds b_o      `bias`
        q (and k) divided by the root mean square over ALL of the token's q (k) numbers, times a weight each
                                                                                        `qk_norm="whole"`
        q, k rotated on the first rotary_dim dims (`position`, either pairing); `qk_norm="unit"`: each head by itself
        q times 1 + coef ln(floor((pos + 1) / every) + 1)                              `q_temp=(coef, every)`
        keys seen: all earlier ones, the last `window`, or those of the row's own run of `chunk` positions
        `maps=2`: two score maps per head (q and k hold [map 1 | map 2] head by head) over the same values,
                  o = a1 - lambda a2, lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff (a scalar of the layer)
        o divided by its root mean square over the head, no weight (`sub_norm`), times `out_scale`
        o times sigmoid(W_g h): one number per head (`gate="head"`) or per element (`gate="element"`)

    The attention kernels work on heads of one size D = max(head_dim, value_dim), rounded up to a multiple of 16
    where that keeps the matrix-core kernels in reach: queries, keys and values are laid out with zeros beyond their
    own sizes (a zero adds nothing to a score, and the values' columns come first in the result), and the two maps
    are two passes of the kernel over caches of their own keys and the one cache of values.  One product reads h for
    [q | k | v | gates] and leaves float32; everything up to the rounded queries and cached keys is float32
    arithmetic in one kernel, everything behind the attention kernel in another.  An output bias is a column of
    the output product's weight that meets a column of ones.  Returns the result by itself in float32 when
    `residual` is None."""
    graph_safe = True
    accepts_lazy_norm = False
    prepares_next_norm = False

    def __init__(self, prefix, dtype, device, *, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 value_dim: int = None, position: dict = None, window: int = 0, chunk: int = 0, scale: float = None,
                 bias: bool = False, out_bias: bool = None, qk_norm: str = None, eps: float = 1e-6, q_temp=None,
                 maps: int = 1, diff: float = 0.0, sub_norm: bool = False, out_scale: float = 1.0, gate: str = None,
                 names: Dict[str, str] = None, bias_suffix: str = ".b", norm_suffix: str = ".norm",
                 max_position: int = 0):
        dim, vdim = int(head_dim), int(value_dim if value_dim is not None else head_dim)
        if dim <= 0 or vdim <= 0:
            raise ValueError(f"{prefix}: head_dim and value_dim must be positive")
        D = max(dim, vdim)
        # a multiple of 16 where the matrix-core kernels take the head (up to 128), else of 8 (rows of 16 bytes)
        D = -(-D // 16) * 16 if -(-D // 16) * 16 <= 128 else -(-D // 8) * 8
        if window and chunk:
            raise ValueError(f"{prefix}: a window or a chunked mask, not both")
        if int(window) < 0 or int(chunk) < 0:
            raise ValueError(f"{prefix}: window and chunk are positive (0: none)")
        super().__init__(prefix, dtype, device, hidden_size=hidden_size, num_heads=num_heads, num_kv_heads=num_kv_heads,
                         head_dim=D, position=None, window=int(window) if window else -int(chunk or 0), scale=1.0)
        if scale is None:
            scale = 1.0 / math.sqrt(dim)
        self.scale = float(scale)
        self.qk_dim, self.value_dim, self.chunk = dim, vdim, int(chunk or 0)
        if qk_norm not in (None, "unit", "whole"):
            raise ValueError(f"{prefix}: qk_norm is None, 'unit' or 'whole', got {qk_norm!r}")
        if maps not in (1, 2):
            raise ValueError(f"{prefix}: one or two score maps, got {maps}")
        if gate not in ops.ATTN_GATES:
            raise ValueError(f"{prefix}: gate is None, 'head' or 'element', got {gate!r}")
        pos = dict(position or {"kind": "none"})
        kind = pos.pop("kind")
        if kind == "rotary":
            pos.setdefault("head_dim", dim)
        self.position = POSITION_ENCODINGS.get(kind)(f"{prefix}.position", dtype, device, **pos)
        self.bias, self.out_bias = bool(bias), bool(bias if out_bias is None else out_bias)
        self.qk_norm, self.eps, self.maps, self.diff = qk_norm, float(eps), int(maps), float(diff)
        self.q_temp = (float(q_temp[0]), int(q_temp[1])) if q_temp else None
        if self.q_temp and self.q_temp[1] <= 0:
            raise ValueError(f"{prefix}: the query temperature's step must be positive")
        self.sub_norm, self.out_scale, self.gate = bool(sub_norm), float(out_scale), gate
        n = {k: k for k in ("q", "k", "v", "g", "o", "lq1", "lk1", "lq2", "lk2")}
        n.update(names or {})
        self.names = {k: f"{prefix}.{v}" for k, v in n.items()}
        self.bias_suffix, self.norm_suffix = bias_suffix, norm_suffix
        H, G = self.num_heads, self.num_kv_heads
        self.q_cols, self.k_cols, self.v_cols = H * self.maps * dim, G * self.maps * dim, G * vdim
        self.q_size = H * D                             # one map's query rows as the attention kernels see them
        self.v_off = self.q_cols + self.k_cols
        self.g_off = -(-(self.v_off + self.v_cols) // 8) * 8
        self.g_cols = {None: 0, "head": H, "element": H * vdim}[gate]
        self.in_width = self.g_off + -(-self.g_cols // 8) * 8
        self.out_cols = H * vdim
        self.out_tail = 8 if self.out_bias else 0       # a column of ones for the bias, zeros up to a multiple of 8
        ops.check_linear_sizes(dtype, self.out_cols, f"{prefix}: num_heads * value_dim")
        self.w_in = self.b_in = self.norm_w = self.w_o = None
        self.lam = 0.0

    def weights(self) -> List[WeightSpec]:
        n, W, bs = self.names, self.hidden_size, self.bias_suffix
        vec = dict(role="vector", init="zeros")
        out = [WeightSpec(n["q"], (self.q_cols, W)), WeightSpec(n["k"], (self.k_cols, W)), WeightSpec(n["v"], (self.v_cols, W))]
        if self.bias:
            out += [WeightSpec(n["q"] + bs, (self.q_cols,), **vec), WeightSpec(n["k"] + bs, (self.k_cols,), **vec),
                    WeightSpec(n["v"] + bs, (self.v_cols,), **vec)]
        if self.qk_norm == "whole":
            out += [WeightSpec(n["q"] + self.norm_suffix, (self.q_cols,), role="vector", init="ones"),
                    WeightSpec(n["k"] + self.norm_suffix, (self.k_cols,), role="vector", init="ones")]
        if self.maps == 2:
            out += [WeightSpec(n[k], (self.qk_dim,), role="vector", init="normal") for k in ("lq1", "lk1", "lq2", "lk2")]
        if self.gate:
            out.append(WeightSpec(n["g"], (self.g_cols, W)))
        out.append(WeightSpec(n["o"], (W, self.out_cols)))
        if self.out_bias:
            out.append(WeightSpec(n["o"] + bs, (W,), **vec))
        return out

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        n, bs = self.names, self.bias_suffix
        dev = tensors[n["q"]].device
        f32 = lambda t: t.to(torch.float32)
        w = torch.zeros((self.in_width, self.hidden_size), dtype=self.dtype, device=dev)
        w[:self.q_cols] = tensors[n["q"]]
        w[self.q_cols:self.v_off] = tensors[n["k"]]
        w[self.v_off:self.v_off + self.v_cols] = tensors[n["v"]]
        if self.gate:
            w[self.g_off:self.g_off + self.g_cols] = tensors[n["g"]]
        self.w_in = w
        if self.bias:
            self.b_in = torch.cat([f32(tensors[n[k] + bs]) for k in ("q", "k", "v")]).contiguous()
        if self.qk_norm == "whole":
            self.norm_w = torch.cat([f32(tensors[n[k] + self.norm_suffix]) for k in ("q", "k")]).contiguous()
        w_o = tensors[n["o"]]
        if self.out_bias:
            wide = torch.zeros((self.hidden_size, self.out_cols + self.out_tail), dtype=self.dtype, device=dev)
            wide[:, :self.out_cols] = w_o
            wide[:, self.out_cols] = tensors[n["o"] + bs]
            w_o = wide
        self.w_o = w_o.contiguous()
        if self.maps == 2:
            # a scalar of the layer, formed once in float32
            l1 = (f32(tensors[n["lq1"]]) * f32(tensors[n["lk1"]])).sum()
            l2 = (f32(tensors[n["lq2"]]) * f32(tensors[n["lk2"]])).sum()
            self.lam = float(torch.exp(l1) - torch.exp(l2)) + self.diff

    def cache_spec(self) -> CacheSpec:
        t = (self.num_kv_heads, self.head_dim)
        kind = "window" if self.window > 0 else "full"
        names = ("k", "k2", "v") if self.maps == 2 else ("k", "v")
        return CacheSpec(tuple(CacheTensor(name, t, 1) for name in names), kind, max(self.window, 0))

    def forward(self, h, ctx, cache: LayerCache, state, residual):
        T, dev, H = h.shape[0], h.device, self.num_heads
        p = ops.scratch("qk_product", (T, self.in_width), torch.float32, dev)
        ops.linear(h, self.w_in, p)
        tables = self.position.rotary_tables()
        cos, sin, rot = tables if tables is not None else (None, None, 0)
        pairing = getattr(self.position, "pairing", "half")
        q = ops.scratch("q_prepared", (self.maps, T, self.q_size), self.dtype, dev)
        write = cache.write
        k_caches = [cache.tensors["k"]] + ([cache.tensors["k2"]] if self.maps == 2 else [])
        ops.attn_prepare(p, self.b_in, self.norm_w, ctx.positions, cos, sin,
                         ctx.slot_mappings[cache.group] if write else None, q, k_caches if write else None,
                         cache.tensors["v"] if write else None, H, self.num_kv_heads, self.maps, self.qk_dim,
                         self.value_dim, self.v_off, rot, pairing, self.qk_norm == "whole", self.qk_norm == "unit",
                         self.eps, self.q_temp)
        outs = []
        for m in range(self.maps):
            # float32 whatever the engine's type: the maps' difference, the head's norm and the gates follow in float32
            attn = ops.scratch("attention_out" if m == 0 else "attention_out2", (T, self.q_size), torch.float32, dev)
            view = LayerCache({"k": k_caches[m], "v": cache.tensors["v"]}, cache.group, cache.write)
            outs.append(self._attend(q[m], ctx, view, attn))
        z = ops.scratch("attention_gated", (T, self.out_cols + self.out_tail), self.dtype, dev)
        gate = p[:, self.g_off:self.g_off + self.g_cols] if self.gate else None
        ops.attn_finish(outs[0], outs[1] if self.maps == 2 else None, gate, z, H, self.value_dim, self.lam, self.sub_norm,
                        self.eps, self.out_scale, self.gate, self.out_tail)
        if residual is None:
            return ops.linear(z, self.w_o, ops.scratch("sublayer_out", (T, self.hidden_size), torch.float32, dev))
        return ops.linear(z, self.w_o, residual, residual)


register_mixer("attention", Attention)
register_mixer("gated_attention", GatedAttention)
register_mixer("normed_attention", NormedAttention)
