"""Mixtures of small feed-forward layers.

`table_moe`: a mixture of small gated feed-forward layers without a router: a table gives every token id its
`top` experts, each with weight 1 / top; an optional shared expert runs for every token and is added,
optionally times sigmoid(w_sg . h), one number per token.

Experts are `clamped_glu` units (parts/mlp.py): down(g * sigmoid(alpha g) * (u + shift)) with
g = min(gate(h), limit), u = clamp(up(h), -limit, limit), without biases.  Their weights are stacked on
load ([E, 2F, W] and [E, W, F]); a step multiplies every token's row with the weights of its own experts.
Tensor names below the prefix: e<i>.gate|up|down, table, shared.gate|up|down, shared.sg.

`routed_moe`: experts down(act(up(h))) without gate or bias, chosen by a router: scores s = softmax(W_router h)
over all experts (float32); the experts lie in `groups` equal runs of neighbours, a run's score is its largest
score and only experts of the `keep` best runs may be chosen; the `top` largest scores among those are chosen and
weigh s_j / (sum of the chosen + 1e-20) * scale; an optional shared expert of the same form runs for every token
and is added.  Tensor names below the prefix: e<i>.up|down, router, shared.up|down.  Options: `activation="swiglu"`
makes the experts gated units down(silu(gate(h)) * up(h)) (tensors e<i>.gate|up|down); `router_bias` adds a bias per
expert to the router's logits (tensor router<bias_suffix>).  With one group and scale 1 the weights are the softmax
over the chosen logits alone: exp(z_j) / sum over the chosen of exp(z_i), whatever the other experts' logits are.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .base import FeedForward, WeightSpec, add_to_residual, register_feed_forward
from .mlp import ActMLP, ClampedGLU


class TableMoE(FeedForward):
    graph_safe = True
    GROUPED_ROWS = 64       # from this many rows (tokens * top) on, a bfloat16 step groups its rows by expert
    RUN_ROWS = 64           # from this many rows an expert on average, the rows are copied into runs of 256 an expert

    def __init__(self, prefix, dtype, device, *, hidden_size: int, vocab_size: int, num_experts: int, top: int,
                 intermediate_size: int, limit: float, alpha: float = 1.702, shift: float = 1.0,
                 shared: Optional[dict] = None):
        """shared: None, or {"intermediate_size": F, "limit": L, "gate": bool} for the shared expert."""
        super().__init__(prefix, dtype, device)
        self.hidden_size, self.vocab_size = int(hidden_size), int(vocab_size)
        self.num_experts, self.top, self.intermediate_size = int(num_experts), int(top), int(intermediate_size)
        self.limit, self.alpha, self.shift = float(limit), float(alpha), float(shift)
        if not (0 < self.top <= self.num_experts):
            raise ValueError(f"{prefix}: a token uses 1 to {self.num_experts} experts, got top = {self.top}")
        if not self.limit > 0:
            raise ValueError(f"{prefix}: the limit of the gated unit must be positive")
        ops.check_linear_sizes(dtype, self.hidden_size, f"{prefix}: hidden_size")
        ops.check_linear_sizes(dtype, self.intermediate_size, f"{prefix}: expert intermediate_size")
        self.shared = None
        self.shared_gate = False
        if shared:
            self.shared = ClampedGLU(f"{prefix}.shared", dtype, device, hidden_size=self.hidden_size,
                                     intermediate_size=int(shared["intermediate_size"]), limit=float(shared["limit"]),
                                     alpha=float(shared.get("alpha", alpha)), shift=float(shared.get("shift", shift)))
            self.shared_gate = bool(shared.get("gate", True))
        self.w_gate_up = self.w_down = self.table = self.w_sg = None

    def weights(self) -> List[WeightSpec]:
        p, W, F = self.prefix, self.hidden_size, self.intermediate_size
        out = []
        for e in range(self.num_experts):
            out += [WeightSpec(f"{p}.e{e}.gate", (F, W)), WeightSpec(f"{p}.e{e}.up", (F, W)),
                    WeightSpec(f"{p}.e{e}.down", (W, F))]
        out.append(WeightSpec(f"{p}.table", (self.vocab_size, self.top), role="table", init=f"distinct:{self.num_experts}"))
        if self.shared is not None:
            out += self.shared.weights()
            if self.shared_gate:
                out.append(WeightSpec(f"{p}.shared.sg", (1, W)))
        return out

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        p, E = self.prefix, self.num_experts
        self.w_gate_up = torch.stack([torch.cat([tensors[f"{p}.e{e}.gate"], tensors[f"{p}.e{e}.up"]], dim=0)
                                      for e in range(E)]).contiguous()
        self.w_down = torch.stack([tensors[f"{p}.e{e}.down"] for e in range(E)]).contiguous()
        table = tensors[f"{p}.table"].to(torch.int32).contiguous()
        if table.numel() and (int(table.min()) < 0 or int(table.max()) >= E):
            raise ValueError(f"{p}.table names experts outside 0 .. {E - 1}")
        self.table = table
        if self.shared is not None:
            self.shared.bind(tensors)
            if self.shared_gate:
                self.w_sg = tensors[f"{p}.shared.sg"].reshape(-1).contiguous()

    def forward(self, h, ctx, residual):
        T, dev, F = h.shape[0], h.device, self.intermediate_size
        tokens = ctx.tokens
        base = scale = None
        if self.shared is not None:
            base = self.shared.forward(h, ctx, None)
            if self.shared_gate:
                scale = ops.row_dot_sigmoid(h, self.w_sg, ops.scratch("moe_shared_gate", (T,), torch.float32, dev))
        rows = T * self.top
        out = base if base is not None else ops.scratch("sublayer_out", (T, self.hidden_size), torch.float32, dev)
        if self.dtype == torch.bfloat16 and rows >= self.RUN_ROWS * self.num_experts:
            # very many rows (prompts): every expert's rows side by side in runs of 256, and the tiled product of
            # the dense layers with a weight matrix per run
            E, R = self.num_experts, ops.MOE_RUN_ROWS
            cap = ops.moe_max_tiles(rows, E, R) * R
            plan = ops.scratch("moe_plan", (ops.moe_plan_ints(rows, E, R),), torch.int32, dev)
            ops.moe_plan(tokens, self.table, plan, E, R)
            runs = ops.moe_tile_experts(plan, rows, E, R)
            hp = ops.scratch("moe_rows_in", (cap, self.hidden_size), self.dtype, dev)
            pos = ops.scratch("moe_row_pos", (rows,), torch.int32, dev)
            ops.moe_gather(h, self.top, plan, rows, E, R, hp, pos)
            gup = ops.scratch("moe_gate_up", (cap, 2 * F), self.dtype, dev)
            ops.linear_grouped(hp, self.w_gate_up, runs, gup)
            zp = ops.scratch("moe_gated", (cap, F), self.dtype, dev)
            ops.clamped_glu(gup, zp, self.limit, self.alpha, self.shift)
            y = ops.scratch("moe_rows_out", (cap, self.hidden_size), torch.float32, dev)
            ops.linear_grouped(zp, self.w_down, runs, y)
            ops.moe_combine_at(y, pos, out, self.top, 1.0 / self.top, base, scale)
        elif self.dtype == torch.bfloat16 and rows >= self.GROUPED_ROWS:
            # many rows: sorted by expert on the device, tiles of one expert's rows on the matrix cores
            gu = ops.scratch("moe_gate_up", (rows, 2 * F), self.dtype, dev)
            z = ops.scratch("moe_gated", (rows, F), self.dtype, dev)
            plan = ops.scratch("moe_plan", (ops.moe_plan_ints(rows, self.num_experts),), torch.int32, dev)
            ops.moe_plan(tokens, self.table, plan, self.num_experts)
            ops.grouped_rows_gemm(h, self.top, self.w_gate_up, plan, gu)
            ops.clamped_glu(gu, z, self.limit, self.alpha, self.shift)
            y = ops.scratch("moe_rows_out", (rows, self.hidden_size), torch.float32, dev)
            ops.grouped_rows_gemm(z, 1, self.w_down, plan, y)
            ops.moe_combine(y, out, self.top, 1.0 / self.top, base, scale)
        else:
            # few rows (decoding) and float32: each row against its own expert's weights
            gu = ops.scratch("moe_gate_up", (rows, 2 * F), self.dtype, dev)
            z = ops.scratch("moe_gated", (rows, F), self.dtype, dev)
            ops.table_moe_up(h, self.w_gate_up, tokens, self.table, gu)
            ops.clamped_glu(gu, z, self.limit, self.alpha, self.shift)
            ops.table_moe_down(z, self.w_down, tokens, self.table, out, 1.0 / self.top, base, scale)
        if residual is None:
            return out
        return add_to_residual(residual, out)


class RoutedMoE(FeedForward):
    graph_safe = True
    GROUPED_ROWS = 64       # from this many rows (tokens * top) on, a bfloat16 step groups its rows by expert
    RUN_ROWS = 64           # from this many rows an expert on average, the rows are copied into runs of 256 an expert

    def __init__(self, prefix, dtype, device, *, hidden_size: int, num_experts: int, top: int, intermediate_size: int,
                 groups: int = 1, keep: int = 1, scale: float = 1.0, activation: str = "relu2",
                 shared: Optional[dict] = None, router_bias: bool = False, bias_suffix: str = ".b"):
        """shared: None, or {"intermediate_size": F} (optionally "activation") for the shared expert."""
        super().__init__(prefix, dtype, device)
        self.hidden_size, self.num_experts, self.top = int(hidden_size), int(num_experts), int(top)
        self.intermediate_size, self.scale = int(intermediate_size), float(scale)
        self.groups, self.keep = max(1, int(groups or 1)), int(keep or 1)
        if not (0 < self.top <= self.num_experts <= ops.MOE_MAX_ROUTED):
            raise ValueError(f"{prefix}: 1 to {ops.MOE_MAX_ROUTED} experts and 1 to all of them a token, got "
                             f"{self.num_experts} and top = {self.top}")
        if self.groups > 1 and (self.num_experts % self.groups or not (0 < self.keep <= self.groups)
                                or self.top > self.keep * (self.num_experts // self.groups)):
            raise ValueError(f"{prefix}: {self.num_experts} experts in {self.groups} groups of which {self.keep} are "
                             f"kept: groups must be equal and the kept ones hold at least top = {self.top} experts")
        self.gated = activation == "swiglu"
        if not self.gated and (activation not in ops.MOE_ACTIVATIONS or activation is None):
            raise ValueError(f"{prefix}: activation {activation!r} is not built; known: relu2, swiglu")
        self.activation = activation
        self.router_bias, self.bias_suffix = bool(router_bias), bias_suffix
        self.b_router = None
        ops.check_linear_sizes(dtype, self.hidden_size, f"{prefix}: hidden_size")
        ops.check_linear_sizes(dtype, self.intermediate_size, f"{prefix}: expert intermediate_size")
        self.shared = None
        if shared:
            self.shared = ActMLP(f"{prefix}.shared", dtype, device, hidden_size=self.hidden_size,
                                 intermediate_size=int(shared["intermediate_size"]),
                                 activation=shared.get("activation", activation))
        self.w_up = self.w_down = self.w_router = None

    def weights(self) -> List[WeightSpec]:
        p, W, F = self.prefix, self.hidden_size, self.intermediate_size
        out = []
        for e in range(self.num_experts):
            if self.gated:
                out.append(WeightSpec(f"{p}.e{e}.gate", (F, W)))
            out += [WeightSpec(f"{p}.e{e}.up", (F, W)), WeightSpec(f"{p}.e{e}.down", (W, F))]
        out.append(WeightSpec(f"{p}.router", (self.num_experts, W)))
        if self.router_bias:
            out.append(WeightSpec(f"{p}.router{self.bias_suffix}", (self.num_experts,), role="vector", init="zeros"))
        if self.shared is not None:
            out += self.shared.weights()
        return out

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        p, E = self.prefix, self.num_experts
        if self.gated:      # an expert's first product gives (gate_0, up_0, gate_1, up_1, ...): rows interleaved, as in
            # the dense gated layer, so that a product's epilogue sees each pair in one lane
            self.w_up = torch.stack([torch.stack([tensors[f"{p}.e{e}.gate"], tensors[f"{p}.e{e}.up"]], dim=1)
                                     .reshape(2 * self.intermediate_size, self.hidden_size) for e in range(E)]).contiguous()
        else:
            self.w_up = torch.stack([tensors[f"{p}.e{e}.up"] for e in range(E)]).contiguous()
        self.w_down = torch.stack([tensors[f"{p}.e{e}.down"] for e in range(E)]).contiguous()
        self.w_router = tensors[f"{p}.router"].contiguous()
        if self.router_bias:
            self.b_router = tensors[f"{p}.router{self.bias_suffix}"].to(torch.float32).contiguous()
        if self.shared is not None:
            self.shared.bind(tensors)
            # one product reads h for the router's logits and the shared expert's hidden units (float32 out):
            # [router, its rows filled up to a multiple of 8 | shared up]
            self.shared_off = -(-E // 8) * 8
            first = torch.zeros((self.shared_off + self.shared.intermediate_size, self.hidden_size), dtype=self.dtype,
                                device=self.w_router.device)
            first[:E] = self.w_router
            first[self.shared_off:] = self.shared.w_up
            self.w_first = first

    def forward(self, h, ctx, residual):
        T, dev, F, E, top = h.shape[0], h.device, self.intermediate_size, self.num_experts, self.top
        # the router: logits, scores and weights in float32
        ids = ops.scratch("moe_ids", (T, top), torch.int32, dev)
        wts = ops.scratch("moe_weights", (T, top), torch.float32, dev)
        if self.shared is not None:
            # with the shared expert's first product; its second one writes the sum the experts are added to
            # (the residual stream itself where the caller gives it)
            Fs = self.shared.intermediate_size
            first = ops.scratch("moe_first", (T, self.shared_off + Fs), torch.float32, dev)
            ops.linear(h, self.w_first, first)
            ops.moe_route(first[:, :E], ids, wts, self.groups, self.keep, self.scale, self.b_router)
            zs = ops.activate_rows(first[:, self.shared_off:], ops.scratch("ffn_gated", (T, Fs), self.dtype, dev),
                                   self.shared.activation)
            if residual is None:
                base = ops.linear(zs, self.shared.w_down, ops.scratch("sublayer_out", (T, self.hidden_size), torch.float32, dev))
            else:
                base = ops.linear(zs, self.shared.w_down, residual, residual)
        else:
            logits = ops.scratch("moe_router", (T, E), torch.float32, dev)
            ops.linear(h, self.w_router, logits)
            ops.moe_route(logits, ids, wts, self.groups, self.keep, self.scale, self.b_router)
            base = residual                     # the experts are added to the stream itself (or stand alone)
        rows = T * top
        out = base if base is not None else ops.scratch("sublayer_out", (T, self.hidden_size), torch.float32, dev)
        if self.dtype == torch.bfloat16 and rows >= self.RUN_ROWS * E:
            # very many rows (prompts): every expert's rows side by side in runs of 256, and the tiled product of
            # the dense layers with a weight matrix per run
            R = ops.MOE_RUN_ROWS
            cap = ops.moe_max_tiles(rows, E, R) * R
            plan = ops.scratch("moe_plan", (ops.moe_plan_ints(rows, E, R),), torch.int32, dev)
            ops.moe_plan(None, ids, plan, E, R, num_tokens=T)
            runs = ops.moe_tile_experts(plan, rows, E, R)
            hp = ops.scratch("moe_rows_in", (cap, self.hidden_size), self.dtype, dev)
            pos = ops.scratch("moe_row_pos", (rows,), torch.int32, dev)
            ops.moe_gather(h, top, plan, rows, E, R, hp, pos)
            z = ops.scratch("moe_gated", (cap, F), self.dtype, dev)
            if self.gated:      # the gate in the product's epilogue
                ops.linear_grouped(hp, self.w_up, runs, z, epilogue="swiglu")
            else:
                up = ops.scratch("moe_up", (cap, F), torch.float32, dev)        # float32: rounded once, behind the activation
                ops.linear_grouped(hp, self.w_up, runs, up)
                ops.activate_rows(up, z, self.activation)
            y = ops.scratch("moe_rows_out", (cap, self.hidden_size), torch.float32, dev)
            ops.linear_grouped(z, self.w_down, runs, y)
            ops.moe_combine_at(y, pos, out, top, 1.0, base, None, wts)
        elif self.dtype == torch.bfloat16 and rows >= self.GROUPED_ROWS:
            # many rows: sorted by expert on the device, tiles of one expert's rows on the matrix cores
            plan = ops.scratch("moe_plan", (ops.moe_plan_ints(rows, E),), torch.int32, dev)
            ops.moe_plan(None, ids, plan, E, num_tokens=T)
            z = ops.scratch("moe_gated", (rows, F), self.dtype, dev)
            if self.gated:
                gup = ops.scratch("moe_gate_up", (rows, 2 * F), self.dtype, dev)
                ops.grouped_rows_gemm(h, top, self.w_up, plan, gup)
                ops.silu_mul(gup, z, pairs=True)
            else:
                up = ops.scratch("moe_up", (rows, F), torch.float32, dev)
                ops.grouped_rows_gemm(h, top, self.w_up, plan, up)
                ops.activate_rows(up, z, self.activation)
            y = ops.scratch("moe_rows_out", (rows, self.hidden_size), torch.float32, dev)
            ops.grouped_rows_gemm(z, 1, self.w_down, plan, y)
            ops.moe_combine(y, out, top, 1.0, base, None, wts)
        else:
            # few rows (decoding) and float32: each row against its own expert's weights, the activation in
            # the first product's kernel
            z = ops.scratch("moe_gated", (rows, F), self.dtype, dev)
            ops.table_moe_up(h, self.w_up, None, ids, z, ops.MOE_GATED if self.gated else self.activation)
            ops.table_moe_down(z, self.w_down, None, ids, out, 1.0, base, None, wts)
        return out


register_feed_forward("table_moe", TableMoE)
register_feed_forward("routed_moe", RoutedMoE)
