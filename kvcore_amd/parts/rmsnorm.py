"""RMSNorm with the residual sum fused in.

Reference: kvcore/model/layer/rmsnorm.py:7-29 (optional add of the residual, float32
square-mean and rsqrt, gain last).  Here the residual stream itself stays float32, so
the sum is never rounded to the model dtype.
"""

from __future__ import annotations

import torch

from kvcore_amd.ops import library as ops

from .base import Norm, ParamSource, ParamSpec, register_norm


class RMSNorm(Norm):
    """``x / sqrt(mean(x^2) + eps) * (weight_offset + weight)``.  ``weight_offset`` 0 is the plain
    norm; 1 serves checkpoints that store the gain as its distance from one.  ``weight_name``: the
    checkpoint tensor relative to the part's prefix (empty: the prefix itself)."""

    def __init__(self, *, hidden_size: int, eps: float, weight_offset: float = 0.0,
                 weight_name: str = "weight") -> None:
        self.hidden_size = hidden_size
        self.eps = eps
        self.weight_offset = float(weight_offset)
        self.weight_name = weight_name
        self._gain: torch.Tensor | None = None

    def param_specs(self) -> list[ParamSpec]:
        return [ParamSpec("weight", (self.hidden_size,), kind="vector",
                          init="normal" if self.weight_offset else "gain",
                          sources=(ParamSource(self.weight_name, 0, self.hidden_size),))]

    def weights_loaded(self) -> None:
        # the gain the kernels multiply by, made once from what the checkpoint stores
        self._gain = self.params["weight"] + self.weight_offset if self.weight_offset else None

    def gain(self) -> torch.Tensor:
        if self.weight_offset and self._gain is None:
            self.weights_loaded()
        return self._gain if self.weight_offset else self.params["weight"]

    def forward_fused(self, out: torch.Tensor, residual: torch.Tensor,
                      delta: torch.Tensor | None) -> None:
        ops.add_rmsnorm(out, residual, delta, self.gain(), self.eps)

    def as_gain(self) -> tuple[torch.Tensor, float]:
        return self.gain(), self.eps

    def forward_rows(self, out: torch.Tensor, x: torch.Tensor) -> None:
        """Normalise rows of ``x`` (model dtype) without a residual."""
        ops.rmsnorm(out, x, self.gain(), self.eps)


register_norm("rmsnorm", RMSNorm)
