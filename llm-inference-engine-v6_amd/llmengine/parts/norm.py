"""RMSNorm: y = w * x / sqrt(mean(x^2) + eps), the weight multiplying directly
(reference: src/kernels.cpp:18-24). Statistics in 32-bit; input is the 32-bit
residual stream, output is in the model's activation type."""
from __future__ import annotations

import torch

from .. import ops
from .base import Getter, Norm, ParamSpec, Placement
from .registry import register_part


class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, size: int, eps: float, tensor: str = "weight"):
        self.size = int(size)
        self.eps = float(eps)
        self.tensor = tensor            # the local name of the weight ("": the part's own name)
        self.weight: torch.Tensor | None = None

    def param_specs(self):
        return {self.tensor: ParamSpec((self.size,), "norm")}

    def load_params(self, get: Getter, placement: Placement) -> None:
        self.weight = placement.place(get(self.tensor))

    def forward(self, x, out, rows=None):
        ops.rmsnorm(x, self.weight, self.eps, out, rows)

    def fused_rms(self):
        # (a subclass that computes something else in `forward` is not this formula any more)
        if type(self).forward is not RMSNorm.forward:
            return None
        return self.weight, self.eps


class CenteredRMSNorm(RMSNorm):
    """RMSNorm whose checkpoint stores the weight's distance from one: y = (1 + w) * x / sqrt(mean(x^2) + eps).
    The sum 1 + w is made once, in 32-bit, when the tensor is loaded; from there on this is the plain formula
    with a 32-bit weight, and every kernel that applies that formula may stand in."""

    def param_specs(self):
        return {self.tensor: ParamSpec((self.size,), "linear")}

    def load_params(self, get: Getter, placement: Placement) -> None:
        self.weight = placement.place(get(self.tensor), torch.float32).add_(1.0)

    def fused_rms(self):
        return self.weight, self.eps


register_part("norm", "rmsnorm", RMSNorm)
register_part("norm", "rmsnorm_centered", CenteredRMSNorm)
