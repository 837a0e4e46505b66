"""The gated delta rule with a decay per head and key channel, or one per head: a recurrent mixer.

Per token (h is the mixer's input, [out, in] weights applied as W h):
    q, k = silu(conv(W_q h)), silu(conv(W_k h))     kv_heads x dim, short causal convolution per channel
    v    = silu(conv(W_v h))                         heads x vdim
    q <- q / sqrt(|q|^2 + 1e-6) * dim^-1/2,  k <- k / sqrt(|k|^2 + 1e-6)       per head
    beta = sigmoid(W_b h)                            per head
    g    = exp(-exp(A_log) * softplus(W_a2 (W_a1 h) + dt_bias))                 heads x dim
    per head:  S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
    out  = W_o concat_heads( w_norm * unit_rms(o) * sigmoid(W_g2 (W_g1 h)) )
Head n reads q/k head n // (heads / kv_heads).  Per request the part keeps S [heads, dim, vdim] and the
last taps - 1 inputs of every convolution, in ONE float32 state row; the cache manager zeroes it when
the request is admitted.  Everything that enters the recurrence is float32 in both precisions.

The products: one reads h for [q | k | v | a1 | g1 | b] (segments start at multiples of 8 columns, the
rows between are zero), one turns [a1 | g1] into [a | g] (a block-diagonal weight: one launch for
the two low-rank products), one is W_o.

Options, each by itself: `decay="head"` (one decay per head: a and dt_bias hold a number per head, every key
channel of the head decays alike), `decay_rank=0` and `gate_rank=0` (the decay's and the gate's pre-activations
come straight from h, `a = W_a h` and `W_g h`; ONE product then reads h for [q | k | v | a | g | b] and leaves
float32), `gate="silu"` (the gate is g * sigmoid(g) instead of the sigmoid).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .base import Mixer, StateSpec, WeightSpec, register_mixer


def _pad8(n: int) -> int:
    return -(-n // 8) * 8


class ChannelDelta(Mixer):
    graph_safe = True

    def __init__(self, prefix, dtype, device, *, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 value_dim: int, conv_taps: int, decay_rank: int, gate_rank: int, eps: float,
                 decay: str = "channel", gate: str = "sigmoid", names: Dict[str, str] = None):
        super().__init__(prefix, dtype, device)
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim, self.value_dim, self.taps = int(head_dim), int(value_dim), int(conv_taps)
        self.decay_rank, self.gate_rank, self.eps = int(decay_rank), int(gate_rank), float(eps)
        ops.check_delta_sizes(self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim, self.taps)
        if decay not in ("channel", "head") or gate not in ("sigmoid", "silu"):
            raise ValueError(f"{prefix}: decay is 'channel' or 'head' and gate 'sigmoid' or 'silu', got {decay!r}, {gate!r}")
        self.per_head, self.gate_kind = decay == "head", gate
        if self.decay_rank < 0 or self.gate_rank < 0 or (self.decay_rank == 0) != (self.gate_rank == 0):
            raise ValueError(f"{prefix}: the decay's and the gate's projections are both low-rank (ranks > 0) or "
                             f"both direct (ranks 0), got {self.decay_rank} and {self.gate_rank}")
        self.direct = self.decay_rank == 0
        ops.check_linear_sizes(dtype, self.hidden_size, f"{prefix}: hidden_size")
        ops.check_linear_sizes(dtype, self.num_heads * self.value_dim, f"{prefix}: heads * value_dim")
        H, KH, D, V = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        self.qk_size, self.v_size = KH * D, H * V
        self.channels = 2 * self.qk_size + self.v_size
        # columns of the product that reads h
        self.low_off = _pad8(self.channels)
        self.n_decay = H if self.per_head else H * D           # pre-activations of the decay per token
        if self.direct:     # [q | k | v | a | g | b]
            self.ra, self.rg = _pad8(self.n_decay), _pad8(H * V)
        else:               # [q | k | v | a1 | g1 | b]
            self.ra, self.rg = _pad8(self.decay_rank), _pad8(self.gate_rank)
        self.b_off = self.low_off + self.ra + self.rg
        self.in_width = self.b_off + _pad8(H)
        self.state_size = H * D * V
        n = {k: k for k in ("q", "k", "v", "b", "A_log", "norm", "a", "a1", "a2", "dt_bias", "g", "g1", "g2", "o")}
        n.update({"q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv"})
        n.update(names or {})
        self.names = {k: f"{prefix}.{v}" for k, v in n.items()}
        self.w_in = self.w_low = self.w_o = None
        self.conv_w = self.a_log = self.dt_bias = self.w_norm = None

    # ---------------------------------------------------------------- declarations
    def weights(self) -> List[WeightSpec]:
        n, W, H, D, V = self.names, self.hidden_size, self.num_heads, self.head_dim, self.value_dim
        vec = dict(role="vector")
        out = [WeightSpec(n["q"], (self.qk_size, W)), WeightSpec(n["q_conv"], (self.qk_size, self.taps), **vec),
               WeightSpec(n["k"], (self.qk_size, W)), WeightSpec(n["k_conv"], (self.qk_size, self.taps), **vec),
               WeightSpec(n["v"], (self.v_size, W)), WeightSpec(n["v_conv"], (self.v_size, self.taps), **vec),
               WeightSpec(n["b"], (H, W)), WeightSpec(n["A_log"], (H,), **vec),
               WeightSpec(n["norm"], (V,), role="vector", init="ones"),
               WeightSpec(n["dt_bias"], (self.n_decay,), **vec)]
        if self.direct:
            out += [WeightSpec(n["a"], (self.n_decay, W)), WeightSpec(n["g"], (H * V, W))]
        else:
            out += [WeightSpec(n["a1"], (self.decay_rank, W)), WeightSpec(n["a2"], (self.n_decay, self.decay_rank)),
                    WeightSpec(n["g1"], (self.gate_rank, W)), WeightSpec(n["g2"], (H * V, self.gate_rank))]
        return out + [WeightSpec(n["o"], (W, H * V))]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        n, H, D, V = self.names, self.num_heads, self.head_dim, self.value_dim
        dev = tensors[n["q"]].device
        w_in = torch.zeros((self.in_width, self.hidden_size), dtype=self.dtype, device=dev)
        at = 0
        for key in ("q", "k", "v"):
            t = tensors[n[key]]
            w_in[at:at + t.shape[0]] = t
            at += t.shape[0]
        first, second = (tensors[n["a"]], tensors[n["g"]]) if self.direct else (tensors[n["a1"]], tensors[n["g1"]])
        w_in[self.low_off:self.low_off + first.shape[0]] = first
        w_in[self.low_off + self.ra:self.low_off + self.ra + second.shape[0]] = second
        w_in[self.b_off:self.b_off + H] = tensors[n["b"]]
        self.w_in = w_in
        if not self.direct:
            w_low = torch.zeros((self.n_decay + H * V, self.ra + self.rg), dtype=self.dtype, device=dev)
            w_low[:self.n_decay, :self.decay_rank] = tensors[n["a2"]]
            w_low[self.n_decay:, self.ra:self.ra + self.gate_rank] = tensors[n["g2"]]
            self.w_low = w_low
        self.w_o = tensors[n["o"]].contiguous()
        f32 = lambda t: t.to(torch.float32).contiguous()
        self.conv_w = torch.cat([f32(tensors[n[k]]) for k in ("q_conv", "k_conv", "v_conv")], dim=0).contiguous()
        self.a_log, self.dt_bias, self.w_norm = f32(tensors[n["A_log"]]), f32(tensors[n["dt_bias"]]), f32(tensors[n["norm"]])

    def state_spec(self) -> StateSpec:
        # a multiple of four floats: rows of the state start at 16-byte boundaries
        return StateSpec((-(-(self.state_size + self.channels * (self.taps - 1)) // 4) * 4,), torch.float32)

    # --------------------------------------------------------------------- compute
    def forward(self, h, ctx, cache, state, residual):
        T, dev = h.shape[0], h.device
        H, KH, D, V = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        if self.direct:
            # every pre-activation straight from h: one product, float32 out
            p = ops.scratch("delta_in", (T, self.in_width), torch.float32, dev)
            ops.linear(h, self.w_in, p)
            a, gate = p[:, self.low_off:self.low_off + self.n_decay], p[:, self.low_off + self.ra:self.low_off + self.ra + H * V]
        else:
            p = ops.scratch("delta_in", (T, self.in_width), self.dtype, dev)
            ops.linear(h, self.w_in, p)
            low = ops.scratch("delta_low", (T, self.n_decay + H * V), torch.float32, dev)
            ops.linear(p[:, self.low_off:self.low_off + self.ra + self.rg], self.w_low, low)
            a, gate = low[:, :self.n_decay], low[:, self.n_decay:]
        z = ops.scratch("delta_gated", (T, H * V), self.dtype, dev)
        if ctx.max_q_len == 1 and T == ctx.num_requests and V <= ops.DELTA_DECODE_MAX_VDIM and V % 4 == 0 \
                and self.taps <= ops.DELTA_DECODE_MAX_TAPS:
            # decoding: every request brings one token; convolutions, recurrence, norm and gate in one kernel
            saved = ops.delta_decode(p, 0, self.b_off, a, gate, self.conv_w, self.a_log, self.dt_bias, self.w_norm, state,
                                     self.state_size, ctx.cu_seqlens_q, ctx.state_slots, z, H, KH, D, V, self.taps,
                                     D ** -0.5, self.eps, self.per_head, self.gate_kind)
            if not saved:       # heads share q/k channels: their saved inputs are shifted behind the kernel
                ops.conv_state_update(p, 0, self.channels, state, self.state_size, ctx.cu_seqlens_q,
                                      ctx.state_slots, self.taps)
            return self._project_out(z, residual)
        qn = ops.scratch("delta_q", (T * H * D,), torch.float32, dev)
        kn = ops.scratch("delta_k", (T * H * D,), torch.float32, dev)
        dec = ops.scratch("delta_decay", (T * H * D,), torch.float32, dev)
        vc = ops.scratch("delta_v", (T * H * V,), torch.float32, dev)
        beta = ops.scratch("delta_beta", (T * H,), torch.float32, dev)
        ops.delta_prepare(p, 0, self.b_off, a, self.conv_w, self.a_log, self.dt_bias, state, self.state_size,
                          ctx.req_of_token, ctx.cu_seqlens_q, ctx.state_slots, qn, kn, vc, beta, dec, H, KH, D, V,
                          self.taps, D ** -0.5, self.per_head)
        ops.conv_state_update(p, 0, self.channels, state, self.state_size, ctx.cu_seqlens_q, ctx.state_slots, self.taps)
        o = ops.scratch("delta_o", (T * H * V,), torch.float32, dev)
        ops.delta_recurrence(qn, kn, vc, beta, dec, state, ctx.cu_seqlens_q, ctx.state_slots, o, H, D, V)
        ops.head_norm_gate(o, self.w_norm, gate, z, H, V, self.eps, self.gate_kind)
        return self._project_out(z, residual)

    def _project_out(self, z, residual):
        if residual is None:
            out = ops.scratch("sublayer_out", (z.shape[0], self.hidden_size), torch.float32, z.device)
            return ops.linear(z, self.w_o, out)
        return ops.linear(z, self.w_o, residual, residual)


register_mixer("channel_delta", ChannelDelta)
