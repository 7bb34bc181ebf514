"""RMSNorm: y = (x / sqrt(mean(x^2) + eps)) * w, computed in float32.

Formula: crates/xrt-kernels/src/cpu/rmsnorm.rs:26-43 of the reference; the
weight is used as stored (not 1 + w).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import Norm, Runtime, WeightSpec, register_part


class RMSNorm(Norm):
    capturable = True

    def __init__(self, prefix: str, dim: int, eps: float):
        self.prefix = prefix
        self.dim = dim
        self.eps = float(eps)
        self.weight = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {self.prefix + "weight": WeightSpec((self.dim,), init="ones", kind="vector")}

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.weight = runtime.vector(tensors[self.prefix + "weight"])

    def row_scale(self):
        return self.weight, self.eps

    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        count = x.shape[0] if rows is None else rows.shape[0]
        out = self.runtime.empty((count, self.dim))
        self.runtime.ops.rmsnorm(x, self.weight, self.eps, out, rows=rows)
        return out


register_part("norm", "rmsnorm", RMSNorm)
