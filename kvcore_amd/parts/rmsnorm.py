"""RMSNorm with the residual sum fused in.

Reference: kvcore/model/layer/rmsnorm.py:7-29 (optional add of the residual, float32
square-mean and rsqrt, gain last).  Here the residual stream itself stays float32, so
the sum is never rounded to the model dtype.
"""

from __future__ import annotations

import torch

from kvcore_amd.ops import library as ops

from .base import Norm, ParamSpec, register_norm


class RMSNorm(Norm):
    def __init__(self, *, hidden_size: int, eps: float) -> None:
        self.hidden_size = hidden_size
        self.eps = eps

    def param_specs(self) -> list[ParamSpec]:
        return [ParamSpec("weight", (self.hidden_size,), kind="vector", init="gain")]

    def forward_fused(self, out: torch.Tensor, residual: torch.Tensor,
                      delta: torch.Tensor | None) -> None:
        ops.add_rmsnorm(out, residual, delta, self.params["weight"], self.eps)

    def as_gain(self) -> tuple[torch.Tensor, float]:
        return self.params["weight"], self.eps

    def forward_rows(self, out: torch.Tensor, x: torch.Tensor) -> None:
        """Normalise rows of ``x`` (model dtype) without a residual."""
        ops.rmsnorm(out, x, self.params["weight"], self.eps)


register_norm("rmsnorm", RMSNorm)
