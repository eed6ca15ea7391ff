"""RMSNorm: ``y = x / sqrt(mean(x^2) + eps) * w`` in 32-bit
(src/model.c:3386-3392; kernel src/kernels.cu:32-48).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import Norm, ParamSpec, register_norm


class RMSNorm(Norm):
    def __init__(self, size: int, eps: float, weight_name: str = "weight", has_weight: bool = True):
        self.size, self.eps = int(size), float(eps)
        self.weight_name, self.has_weight = weight_name, has_weight
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        if not self.has_weight:
            return {}
        return {self.weight_name: ParamSpec((self.size,), role="vector", init="ones_jitter")}

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        self.weight = tensors.get(self.weight_name)

    def forward(self, ctx, x, rows=None):
        return self.rt.ops.rmsnorm(x, self.weight, self.eps, self.rt.dtype, rows=rows)

    def fold(self):
        return (self.weight, self.eps) if self.weight is not None else None


register_norm("rmsnorm", RMSNorm)
