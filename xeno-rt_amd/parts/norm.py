"""RMSNorm: y = (x / sqrt(mean(x^2) + eps)) * w, computed in float32.

Formula: crates/xrt-kernels/src/cpu/rmsnorm.rs:26-43 of the reference; the
weight is used as stored (not 1 + w).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import Norm, Runtime, WeightSpec, register_part


class Normed:
    """The rows of a float32 tensor that are still to be normalised.

    A block hands this to a part whose first operation is a product; the product then takes
    the norm along (one kernel instead of two). `tensor()` normalises now, for any other use.
    """

    def __init__(self, norm: "RMSNorm", x: torch.Tensor, rows: Optional[torch.Tensor] = None):
        self.norm = norm
        self.x = x
        self.rows = rows
        self.shape = (x.shape[0] if rows is None else rows.shape[0], norm.dim)
        self._tensor = None

    def tensor(self) -> torch.Tensor:
        if self._tensor is None:
            self._tensor = self.norm.forward(self.x, rows=self.rows)
        return self._tensor


def linear(runtime: Runtime, h, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> None:
    """out (+)= h . w^T, where h is a tensor or a `Normed`."""
    if isinstance(h, Normed) and not accumulate:
        runtime.ops.norm_linear(h.x, h.norm.weight, h.norm.eps, w, out, gated=False, rows=h.rows)
    else:
        runtime.ops.linear(h.tensor() if isinstance(h, Normed) else h, w, out, accumulate=accumulate)


def linear_glu(runtime: Runtime, h, w_gate_up: torch.Tensor, out: torch.Tensor) -> None:
    """out = silu(h . gate^T) * (h . up^T), where h is a tensor or a `Normed`."""
    if isinstance(h, Normed):
        runtime.ops.norm_linear(h.x, h.norm.weight, h.norm.eps, w_gate_up, out, gated=True, rows=h.rows)
    else:
        runtime.ops.linear_glu(h, w_gate_up, out)


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

    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        count = x.shape[0] if rows is None else rows.shape[0]
        out = self.runtime.empty((count, self.dim))
        self.runtime.ops.rmsnorm(x, self.weight, self.eps, out, rows=rows)
        return out


    def lazy(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> Normed:
        """For parts that say `takes_normed`: the norm is applied inside their first product."""
        return Normed(self, x, rows)


register_part("norm", "rmsnorm", RMSNorm)
