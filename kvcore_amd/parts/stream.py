"""Changes of the whole residual stream between layers.

``LoopInject`` opens a pass of a looped stretch of layers: the stream and the embedding's
output side by side go through one matrix, ``x <- W [x; x0]``, and a vector that belongs to
the pass is added, ``x <- x + step[pass]``.  The product takes its operands in the model
dtype and leaves float32 sums in the stream.
"""

from __future__ import annotations

import torch

from kvcore_amd.ops import library as ops

from .base import ParamSource, ParamSpec, StreamOp, register_stream_op


class LoopInject(StreamOp):
    needs_embedded = True

    def __init__(self, *, hidden_size: int, passes: int, weight_name: str = "in",
                 step_name: str = "step") -> None:
        self.hidden_size = hidden_size
        self.passes = passes
        self.weight_name = weight_name
        self.step_name = step_name

    def param_specs(self) -> list[ParamSpec]:
        H = self.hidden_size
        return [
            ParamSpec("weight", (H, 2 * H), sources=(ParamSource(self.weight_name, 0, H),)),
            ParamSpec("step", (self.passes, H), kind="vector", init="normal",
                      sources=(ParamSource(self.step_name, 0, self.passes),)),
        ]

    def product_weights(self) -> tuple[str, ...]:
        return ("weight",)

    def forward(self, residual: torch.Tensor, embedded: torch.Tensor | None, ctx, arg: int) -> None:
        if embedded is None:
            raise RuntimeError("LoopInject needs the embedding's output")
        if not 0 <= arg < self.passes:
            raise ValueError(f"pass {arg} of {self.passes}")
        H = self.hidden_size
        both = ctx.buf("loop_both", 2 * H)
        ops.concat2(both, residual, embedded)
        ops.linear(residual, both, self.params["weight"])
        ops.add_row(residual, self.params["step"][arg])


register_stream_op("loop_inject", LoopInject)
