"""SwiGLU feed-forward: down( silu(gate(h)) * up(h) ), residual add folded in.

Reference: tiny_llm/parser/llama_parser.cpp:225-255 (gate, SiLU in place, up,
multiply, down, add), tiny_llm/ops/cuda/silu.cu:10 (x / (1 + exp(-x))).  Gate and
up weights are interleaved row by row on load into one [2I, H] matrix, and the
SiLU-gate runs in the epilogue of that one product on its float32 accumulators:
the [T, 2I] intermediate of the reference's four kernels is never written.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .norm import LazyNorm
from .base import FeedForward, WeightSpec, project_into_residual, register_feed_forward


class SwiGLU(FeedForward):
    graph_safe = True
    accepts_lazy_norm = True
    prepares_next_norm = True

    def __init__(self, prefix, dtype, device, *, hidden_size: int, intermediate_size: int):
        super().__init__(prefix, dtype, device)
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        ops.check_linear_sizes(dtype, self.hidden_size, f"{prefix}: hidden_size")
        ops.check_linear_sizes(dtype, self.intermediate_size, f"{prefix}: intermediate_size")
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def weights(self) -> List[WeightSpec]:
        p, H, I = self.prefix, self.hidden_size, self.intermediate_size
        return [WeightSpec(f"{p}.gate_proj.weight", (I, H)), WeightSpec(f"{p}.up_proj.weight", (I, H)),
                WeightSpec(f"{p}.down_proj.weight", (H, I))]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        p = self.prefix
        gate, up = tensors[f"{p}.gate_proj.weight"], tensors[f"{p}.up_proj.weight"]
        # rows interleaved (gate_0, up_0, gate_1, up_1, ...): a product's epilogue then sees each
        # pair side by side and writes silu(gate) * up directly
        self.w_gate_up = torch.stack([gate, up], dim=1).reshape(2 * self.intermediate_size,
                                                                self.hidden_size).contiguous()
        self.w_down = tensors[f"{p}.down_proj.weight"].contiguous()

    def forward(self, h, ctx, residual, next_norm=None):
        T, dev = residual.shape[0], residual.device
        z = ops.scratch("ffn_gated", (T, self.intermediate_size), self.dtype, dev)
        if isinstance(h, LazyNorm):
            h.linear(self.w_gate_up, z, epilogue="swiglu")
        else:
            ops.linear(h, self.w_gate_up, z, epilogue="swiglu")
        out, prepared = project_into_residual(z, self.w_down, residual, next_norm)
        return out if next_norm is None else (out, prepared)


class ClampedGLU(FeedForward):
    """down(g * sigmoid(alpha * g) * (u + shift)) with g = min(gate(h), limit) and
    u = clamp(up(h), -limit, limit).  Gate and up weights are stacked on load into one [2F, H]
    matrix (one product); the activation runs on its result in the engine's element type.

    `names`: the tensors' names below the prefix, (gate, up, down).  With `residual=None` the
    result is returned by itself in float32 (a block that norms the sublayer's output adds it)."""
    graph_safe = True

    def __init__(self, prefix, dtype, device, *, hidden_size: int, intermediate_size: int, limit: float,
                 alpha: float = 1.702, shift: float = 1.0, names=("gate", "up", "down")):
        super().__init__(prefix, dtype, device)
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.limit, self.alpha, self.shift = float(limit), float(alpha), float(shift)
        if not self.limit > 0:
            raise ValueError(f"{prefix}: the limit of the gated unit must be positive")
        ops.check_linear_sizes(dtype, self.hidden_size, f"{prefix}: hidden_size")
        ops.check_linear_sizes(dtype, self.intermediate_size, f"{prefix}: intermediate_size")
        self.names = tuple(f"{prefix}.{n}" for n in names)
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def weights(self) -> List[WeightSpec]:
        H, I = self.hidden_size, self.intermediate_size
        gate, up, down = self.names
        return [WeightSpec(gate, (I, H)), WeightSpec(up, (I, H)), WeightSpec(down, (H, I))]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        gate, up, down = self.names
        self.w_gate_up = torch.cat([tensors[gate], tensors[up]], dim=0).contiguous()
        self.w_down = tensors[down].contiguous()

    def forward(self, h, ctx, residual):
        T, dev = h.shape[0], h.device
        gu = ops.scratch("ffn_gate_up", (T, 2 * self.intermediate_size), self.dtype, dev)
        ops.linear(h, self.w_gate_up, gu)
        z = ops.scratch("ffn_gated", (T, self.intermediate_size), self.dtype, dev)
        ops.clamped_glu(gu, z, self.limit, self.alpha, self.shift)
        if residual is None:
            return ops.linear(z, self.w_down, ops.scratch("sublayer_out", (T, self.hidden_size), torch.float32, dev))
        return ops.linear(z, self.w_down, residual, residual)


class GeluGLU(FeedForward):
    """down(gelu(gate(h)) * up(h)), gelu in its tanh form.  Gate and up weights are stacked on load into
    one [2F, H] matrix (one product); the activation runs on its result in the engine's element type.
    `names`: the tensors' names below the prefix, (gate, up, down).  With `residual=None` the result is
    returned by itself in float32."""
    graph_safe = True

    def __init__(self, prefix, dtype, device, *, hidden_size: int, intermediate_size: int,
                 names=("gate", "up", "down")):
        super().__init__(prefix, dtype, device)
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        ops.check_linear_sizes(dtype, self.hidden_size, f"{prefix}: hidden_size")
        ops.check_linear_sizes(dtype, self.intermediate_size, f"{prefix}: intermediate_size")
        self.names = tuple(f"{prefix}.{n}" for n in names)
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def weights(self) -> List[WeightSpec]:
        H, I = self.hidden_size, self.intermediate_size
        gate, up, down = self.names
        return [WeightSpec(gate, (I, H)), WeightSpec(up, (I, H)), WeightSpec(down, (H, I))]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        gate, up, down = self.names
        self.w_gate_up = torch.cat([tensors[gate], tensors[up]], dim=0).contiguous()
        self.w_down = tensors[down].contiguous()

    def forward(self, h, ctx, residual):
        T, dev = h.shape[0], h.device
        gu = ops.scratch("ffn_gate_up", (T, 2 * self.intermediate_size), self.dtype, dev)
        ops.linear(h, self.w_gate_up, gu)
        z = ops.scratch("ffn_gated", (T, self.intermediate_size), self.dtype, dev)
        ops.gelu_glu(gu, z)
        if residual is None:
            return ops.linear(z, self.w_down, ops.scratch("sublayer_out", (T, self.hidden_size), torch.float32, dev))
        return ops.linear(z, self.w_down, residual, residual)


class ActMLP(FeedForward):
    """down(act(up(h))): a feed-forward without a gate.  act "relu2" is the square of max(., 0).  The up
    product leaves float32 and the activation rounds once to the engine's element type for the down
    product.  `names`: the tensors' names below the prefix, (up, down).  With `residual=None` the result
    is returned by itself in float32."""
    graph_safe = True

    def __init__(self, prefix, dtype, device, *, hidden_size: int, intermediate_size: int, activation: str = "relu2",
                 names=("up", "down")):
        super().__init__(prefix, dtype, device)
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        if activation not in ops.MOE_ACTIVATIONS or activation is None:
            raise ValueError(f"{prefix}: activation {activation!r} is not built; known: relu2")
        self.activation = activation
        ops.check_linear_sizes(dtype, self.hidden_size, f"{prefix}: hidden_size")
        ops.check_linear_sizes(dtype, self.intermediate_size, f"{prefix}: intermediate_size")
        self.names = tuple(f"{prefix}.{n}" for n in names)
        self.w_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def weights(self) -> List[WeightSpec]:
        H, I = self.hidden_size, self.intermediate_size
        up, down = self.names
        return [WeightSpec(up, (I, H)), WeightSpec(down, (H, I))]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        up, down = self.names
        self.w_up = tensors[up].contiguous()
        self.w_down = tensors[down].contiguous()

    def forward(self, h, ctx, residual):
        T, dev = h.shape[0], h.device
        u = ops.scratch("ffn_up", (T, self.intermediate_size), torch.float32, dev)
        ops.linear(h, self.w_up, u)
        z = ops.scratch("ffn_gated", (T, self.intermediate_size), self.dtype, dev)
        ops.activate_rows(u, z, self.activation)
        if residual is None:
            return ops.linear(z, self.w_down, ops.scratch("sublayer_out", (T, self.hidden_size), torch.float32, dev))
        return ops.linear(z, self.w_down, residual, residual)


register_feed_forward("swiglu", SwiGLU)
register_feed_forward("act_mlp", ActMLP)
register_feed_forward("gelu_glu", GeluGLU)
register_feed_forward("clamped_glu", ClampedGLU)
