"""Parts that act on the residual stream between layer runs.

`loop_join`: ahead of every pass through a run of layers that a model repeats with the same weights,
    x <- W_in [x ; x0] + step[turn]
with x0 the embedding's output of the step, W_in [hidden, 2 hidden] (x's columns first) and one vector per pass
(`step` [times, hidden]).  Two launches: one writes the operand [x | x0] in the engine's element type and fills the
new stream's rows with the pass's vector, the product then adds W_in [x ; x0] to them in float32.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .base import StreamPart, WeightSpec, register_stream_part


class LoopJoin(StreamPart):
    graph_safe = True

    def __init__(self, prefix, dtype, device, *, hidden_size: int, times: int, in_name: str = "in",
                 step_name: str = "step"):
        super().__init__(prefix, dtype, device)
        self.hidden_size, self.times = int(hidden_size), int(times)
        if self.times <= 0:
            raise ValueError(f"{prefix}: a repeated run of layers runs at least once, got times = {self.times}")
        ops.check_linear_sizes(dtype, 2 * self.hidden_size, f"{prefix}: 2 * hidden_size")
        self.in_name, self.step_name = f"{prefix}.{in_name}", f"{prefix}.{step_name}"
        self.w_in: Optional[torch.Tensor] = None
        self.steps: Optional[torch.Tensor] = None

    def weights(self) -> List[WeightSpec]:
        W = self.hidden_size
        return [WeightSpec(self.in_name, (W, 2 * W)), WeightSpec(self.step_name, (self.times, W), role="vector")]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.w_in = tensors[self.in_name].contiguous()
        self.steps = tensors[self.step_name].to(torch.float32).contiguous()

    def forward(self, x, origin, ctx, turn: int):
        if not (0 <= turn < self.times):
            raise ValueError(f"{self.prefix}: pass {turn} of {self.times}")
        T, W = x.shape
        operand = ops.scratch("loop_operand", (T, 2 * W), self.dtype, x.device)
        # the stream goes on in a buffer that is not the embedding's output, which later passes still read
        out = x if x.data_ptr() != origin.data_ptr() else ops.scratch("loop_stream", (T, W), torch.float32, x.device)
        ops.stream_join(x, origin, self.steps[turn], operand, out)
        return ops.linear(operand, self.w_in, out, out)


register_stream_part("loop_join", LoopJoin)
