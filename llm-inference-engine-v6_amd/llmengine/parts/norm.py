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

    def __init__(self, size: int, eps: float):
        self.size = int(size)
        self.eps = float(eps)
        self.weight: torch.Tensor | None = None

    def param_specs(self):
        return {"weight": ParamSpec((self.size,), "norm")}

    def load_params(self, get: Getter, placement: Placement) -> None:
        self.weight = placement.place(get("weight"))

    def forward(self, x, out, rows=None):
        ops.rmsnorm(x, self.weight, self.eps, out, rows)

    def fused_rms(self):
        # (a subclass that computes something else in `forward` is not this formula any more)
        if type(self).forward is not RMSNorm.forward:
            return None
        return self.weight, self.eps


register_part("norm", "rmsnorm", RMSNorm)
