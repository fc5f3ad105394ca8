"""Layer norm with weight and bias and the residual sum fused in.

``(x - mean) / sqrt(var + eps) * weight + bias`` over a row, the variance being the mean of the
squared deviations, all in float32 on the float32 residual stream.  It has no form as a bare
gain, so the products around it do none of its work: ``as_gain`` stays None.
"""

from __future__ import annotations

import torch

from kvcore_amd.ops import library as ops

from .base import Norm, ParamSource, ParamSpec, register_norm


class LayerNorm(Norm):
    """``weight_name`` and ``bias_name`` are the checkpoint tensors relative to the part's
    prefix (an empty name is the prefix itself); ``bias`` False leaves the shift out."""

    def __init__(self, *, hidden_size: int, eps: float, bias: bool = True,
                 weight_name: str = "weight", bias_name: str = "bias") -> None:
        self.hidden_size = hidden_size
        self.eps = eps
        self.bias = bias
        self.weight_name = weight_name
        self.bias_name = bias_name

    def param_specs(self) -> list[ParamSpec]:
        H = self.hidden_size
        specs = [ParamSpec("weight", (H,), kind="vector", init="gain",
                           sources=(ParamSource(self.weight_name, 0, H),))]
        if self.bias:
            specs.append(ParamSpec("bias", (H,), kind="vector", init="normal",
                                   sources=(ParamSource(self.bias_name, 0, H),)))
        return specs

    def forward_fused(self, out: torch.Tensor, residual: torch.Tensor,
                      delta: torch.Tensor | None) -> None:
        ops.add_layernorm(out, residual, delta, self.params["weight"], self.params.get("bias"), self.eps)


register_norm("layernorm", LayerNorm)
