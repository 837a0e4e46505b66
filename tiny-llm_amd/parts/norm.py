"""RMSNorm: y = w * x / sqrt(mean(x^2) + eps), statistics in float32.

Reference: tiny_llm/ops/cuda/norm.cu:29-48 (weight applied before the division,
plain `w`, not `1 + w`); placed by tiny_llm/parser/llama_parser.cpp:198-203,
219-224, 258-263.  Unlike the reference (norm.cu:66-85) any width is taken.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .base import ChannelScale, Norm, WeightSpec, register_norm, register_scale


class LazyNorm:
    """A norm that has not run yet: (x, weight, eps).  A consumer that can fuse the norm into its
    first product takes the fields; any other calls `materialize()`.

    `prepared` = (operand, sumsq): the product that wrote x has already written
    operand = bf16(weight * x) and the sums of x^2 over groups of columns
    (`ops.linear_handoff`), so the consumer's product needs no pass over x at all."""

    def __init__(self, norm: "RMSNorm", x: torch.Tensor, rows: Optional[torch.Tensor] = None, prepared=None):
        self.norm, self.x, self.rows = norm, x, rows
        self.weight, self.eps = norm.weight, norm.eps
        self.prepared = prepared

    def linear(self, w: torch.Tensor, out: torch.Tensor, epilogue: Optional[str] = None) -> torch.Tensor:
        """out = norm(x)[rows] @ w.T (then the epilogue), by the cheapest route there is."""
        if self.x.dtype == torch.float32 and w.dtype == torch.float32:
            # true float32: the norm inside the few-row product's kernel (measured on whole steps: up
            # to 16 rows it saves time), or as two kernels that give the same bits: norm_weight * x
            # and the rows' factors, then the product with the factor applied to its sums
            # (a product so wide that a workgroup owns several column tiles takes the two kernels too)
            if (self.rows is None and self.x.shape[0] <= RMSNorm.F32_FUSED_ROWS
                    and ops.linear_norm_f32_ok(self.x.shape[0], w.shape[0], self.x.shape[1], self.x.stride(0))
                    and ops.linear_f32_col_tiles(self.x.shape[0], w.shape[0], self.x.shape[1]) == 1):
                return ops.linear_norm_f32(self.x, self.weight, self.eps, w, out, epilogue=epilogue)
            h, inv_rms = ops.norm_prescale_f32(self.x, self.weight, self.eps, self.rows)
            return ops.linear(h, w, out, epilogue=epilogue, row_scale=inv_rms)
        if self.prepared is not None and (self.num_rows <= ops.FEW_ROWS or self.rows is None):
            operand, sumsq = self.prepared
            return ops.linear_handoff(operand, w, out, epilogue=epilogue, rows=self.rows,
                                      prepared=(sumsq, self.eps, self.x.shape[1]))
        return ops.linear_norm(self.x, self.weight, self.eps, w, out, rows=self.rows, epilogue=epilogue)

    @property
    def num_rows(self) -> int:
        return self.x.shape[0] if self.rows is None else self.rows.numel()

    def materialize(self) -> torch.Tensor:
        return self.norm.forward(self.x, self.rows)


class RMSNorm(Norm):
    graph_safe = True
    F32_FUSED_ROWS = 16      # measured on whole steps: beyond, the norm's own kernel is as fast or faster

    def __init__(self, prefix, dtype, device, *, hidden_size: int, eps: float, init: str = "ones",
                 offset: float = 0.0, weight_name: str = "weight"):
        """offset: the effective weight is offset + the stored one (1.0 for checkpoints that store
        the weight around zero); it is then kept in float32.  weight_name: the tensor's name below
        the prefix ("" if the prefix itself names it)."""
        super().__init__(prefix, dtype, device)
        self.hidden_size = int(hidden_size)
        self.eps = float(eps)
        self.offset = float(offset)
        self.init = init if not self.offset else "zeros"
        self.tensor_name = f"{prefix}.{weight_name}" if weight_name else prefix
        self.weight: Optional[torch.Tensor] = None

    def weights(self) -> List[WeightSpec]:
        return [WeightSpec(self.tensor_name, (self.hidden_size,), role="vector", init=self.init)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        w = tensors[self.tensor_name]
        # offset + w is formed in float32: in bfloat16 the sum would lose what the stored weight says
        self.weight = (w.to(torch.float32) + self.offset).contiguous() if self.offset else w.contiguous()

    def add_normed(self, y: torch.Tensor, x: torch.Tensor, scale: Optional[torch.Tensor] = None,
                   copy: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x += scale * norm(y) for a norm that sits on a sublayer's output (y float32, one kernel);
        `copy` receives the new x in its own element type."""
        w = self.weight if self.weight.dtype == torch.float32 else self.weight.to(torch.float32)
        return ops.norm_scale_add(y, w, self.eps, x, scale, copy)

    def lazy(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None, prepared=None):
        """The norm rides in the consumer's first product: in bfloat16 always (`ops.linear_norm`), in
        float32 for at most 16 rows (`ops.linear_norm_f32`); more rows, or gathered rows, get the
        norm as a row factor of the product (`ops.norm_prescale_f32`), which gives the same bits."""
        if self.dtype == torch.bfloat16 and self.hidden_size % 8 == 0:
            return LazyNorm(self, x, rows, prepared)
        if self.dtype == torch.float32 and self.weight.dtype == torch.float32:
            return LazyNorm(self, x, rows, None)
        return self.forward(x, rows)

    def hand_off_buffers(self, n_rows: int, inner: int, device):
        """(weight, operand, sumsq) for a product (inner size `inner`) that writes this norm's input
        and can prepare the norm on the way (`ops.linear_handoff`), or None where that does not apply."""
        if not ops.can_hand_off(n_rows, self.hidden_size, inner, self.dtype):
            return None
        # still read by the next product while the product after that writes its own: three in turn
        operand = ops.scratch("handoff_operand", (n_rows, self.hidden_size), torch.bfloat16, device, rotate=3)
        sumsq = ops.scratch("handoff_sumsq", (n_rows, ops.handoff_parts(n_rows, self.hidden_size, inner)),
                            torch.float32, device, rotate=3)
        return self.weight, operand, sumsq

    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        n = x.shape[0] if rows is None else rows.numel()
        # two in turn: a block's second norm is computed while nothing reads its first any more, but
        # the final norm's rows must not alias what a consumer still holds
        out = ops.scratch("normed", (n, self.hidden_size), self.dtype, x.device, rotate=2)
        return ops.rmsnorm(x, self.weight, self.eps, out, rows)


class LayerNorm(Norm):
    """(x - mean) / sqrt(var + eps) * w + b over a row, var the mean squared deviation; statistics, weight
    and bias in float32.  `weight_name` / `bias_name`: the tensors' names below the prefix ("" for the
    prefix itself).  `sum_normed` serves a layer whose norm FOLLOWS the sum: x <- LN(alpha * x + y); `add_scaled_norm` one
    whose norm sits on the sublayer's result: x <- x + mult * LN(y)."""
    graph_safe = True

    def __init__(self, prefix, dtype, device, *, hidden_size: int, eps: float, weight_name: str = "weight",
                 bias_name: str = "bias"):
        super().__init__(prefix, dtype, device)
        self.hidden_size = int(hidden_size)
        self.eps = float(eps)
        if not self.eps > 0:
            raise ValueError(f"{prefix}: eps must be positive")
        self.weight_name = f"{prefix}.{weight_name}" if weight_name else prefix
        self.bias_name = f"{prefix}.{bias_name}" if bias_name else prefix
        if self.weight_name == self.bias_name:
            raise ValueError(f"{prefix}: weight and bias need two tensor names")
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    def weights(self) -> List[WeightSpec]:
        return [WeightSpec(self.weight_name, (self.hidden_size,), role="vector", init="ones"),
                WeightSpec(self.bias_name, (self.hidden_size,), role="vector", init="zeros")]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.weight_name].to(torch.float32).contiguous()
        self.bias = tensors[self.bias_name].to(torch.float32).contiguous()

    def sum_normed(self, y: Optional[torch.Tensor], x: torch.Tensor, alpha: float,
                   copy: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x <- LN(alpha * x + y) in place (y float32 or None, one kernel); `copy` receives the new x in
        its own element type."""
        return ops.layer_norm_sum(y, self.weight, self.bias, x, alpha, self.eps, copy)

    def add_scaled_norm(self, y: torch.Tensor, x: torch.Tensor, mult: float = 1.0, then: "LayerNorm" = None):
        """x <- x + mult * LN(y) in place, for a norm that sits on a sublayer's result (y float32, one kernel).
        `then`: the layer norm that reads the new x next; its result comes out of the same kernel and is returned
        (None without one, or where the kernel does not take the width)."""
        if self.hidden_size > ops.LAYER_NORM_ADD_MAX:
            raise ValueError(f"{self.prefix}: a layer norm behind a sublayer takes rows of at most {ops.LAYER_NORM_ADD_MAX}")
        if then is None:
            ops.layer_norm_add(y, self.weight, self.bias, x, mult, self.eps)
            return None
        out = ops.scratch("normed", x.shape, then.dtype, x.device, rotate=2)
        ops.layer_norm_add(y, self.weight, self.bias, x, mult, self.eps, then=(then.weight, then.bias, then.eps, out))
        return out

    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        n = x.shape[0] if rows is None else rows.numel()
        out = ops.scratch("normed", (n, self.hidden_size), self.dtype, x.device, rotate=2)
        return ops.layer_norm_rows(x, self.weight, self.bias, self.eps, out, rows)


class VectorScale(ChannelScale):
    """A learned vector that multiplies a sublayer's result channel by channel; kept in float32.
    The tensor is named by the prefix itself."""
    graph_safe = True

    def __init__(self, prefix, dtype, device, *, hidden_size: int):
        super().__init__(prefix, dtype, device)
        self.hidden_size = int(hidden_size)
        self.weight: Optional[torch.Tensor] = None

    def weights(self) -> List[WeightSpec]:
        return [WeightSpec(self.prefix, (self.hidden_size,), role="vector", init="ones")]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.prefix].to(torch.float32).contiguous()


register_norm("rmsnorm", RMSNorm)
register_norm("layernorm", LayerNorm)
register_scale("vector", VectorScale)
