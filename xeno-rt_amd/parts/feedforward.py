"""Dense gated feed-forward: x + W_down (act(W_gate y) * (W_up y)), no biases.

The reference's SwiGLU block (crates/xrt-models/src/llama.rs:582-601) with
silu(z) = z / (1 + exp(-z)) (crates/xrt-kernels/src/cpu/silu.rs:1-3, 22-24).
Gate and up are bound as one matrix [2I][H] so that one product reads the
normed activations once, as the reference fuses the two dispatches
(llama.rs:584-594).
"""
from __future__ import annotations

from typing import Dict

import torch

from .base import FeedForward, Runtime, WeightSpec, register_part


class GatedMLP(FeedForward):
    capturable = True
    passes_norms = True

    ACTIVATIONS = ("silu",)

    def __init__(self, prefix: str, hidden: int, intermediate: int, activation: str = "silu"):
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"activation must be one of {self.ACTIVATIONS}, found {activation!r}")
        self.prefix = prefix
        self.hidden = hidden
        self.intermediate = intermediate
        self.activation = activation
        self.w_gate_up = None
        self.w_down = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, h, i = self.prefix, self.hidden, self.intermediate
        return {
            p + "gate_proj.weight": WeightSpec((i, h)),
            p + "up_proj.weight": WeightSpec((i, h)),
            p + "down_proj.weight": WeightSpec((h, i)),
        }

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        p = self.prefix
        self.w_gate_up = runtime.weight([tensors[p + name] for name in ("gate_proj.weight", "up_proj.weight")],
                                        "gated", gated_n=self.intermediate)
        self.w_down = runtime.weight(tensors[p + "down_proj.weight"])

    def forward(self, h, batch, residual: torch.Tensor, then=None):
        rt = self.runtime
        tokens = h.shape[0]
        act = rt.empty((tokens, self.intermediate))
        rt.ops.linear_glu(h, self.w_gate_up, act, activation=self.activation)
        return rt.ops.linear(act, self.w_down, residual, accumulate=True,
                             then_norm=None if then is None else then.row_scale())


register_part("feed_forward", "gated_mlp", GatedMLP)
