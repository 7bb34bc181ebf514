"""Position encodings applied to queries and keys before the keys are cached.

Rotary: pairs (i, i + rope_dim/2) of every head are rotated by the angle
pos * scale / theta_i with theta_i = base^(2i/rope_dim); formulas of the
reference's crates/xrt-kernels/src/cpu/rope.rs:10-16 (table), :59-68 (angle),
:71-89 (rotation). Table, angle, sine and cosine are float32.
"""
from __future__ import annotations

import torch

from .base import HalfSplitRotation, PositionEncoding, Runtime, register_part


class Rotary(PositionEncoding):
    capturable = True

    def __init__(self, rope_dim: int, base: float, scale: float = 1.0, table_positions: int = 0):
        """table_positions: positions (from 0 on) whose cosines and sines are worked out once, when the part is bound,
        for kernels that can read them (a decode step's attention, where it also finishes q and k); 0: none."""
        if rope_dim <= 0 or rope_dim % 2 != 0:
            raise ValueError(f"rotary width must be positive and even, found {rope_dim}")
        self.rope_dim = rope_dim
        self.base = float(base)
        self.scale = float(scale)
        self.table_positions = int(table_positions)
        self.theta = None
        self.table = None

    def bind(self, tensors, runtime: Runtime) -> None:
        if self.theta is not None and getattr(self, "runtime", None) is runtime:
            return                                  # one encoding may serve many mixers: bound once
        super().bind(tensors, runtime)
        pair = torch.arange(self.rope_dim // 2, dtype=torch.float32)
        # float32 power, like the reference's powf (rope.rs:13)
        theta = torch.tensor(self.base, dtype=torch.float32) ** ((2.0 * pair) / float(self.rope_dim))
        self.theta = theta.to(runtime.device)
        make_table = getattr(runtime.ops, "rope_table", None)
        if self.table_positions > 0 and make_table is not None and self.theta.device.type == "cuda":
            self.table = make_table(self.theta, self.rope_dim, self.scale, self.table_positions)

    def rotation(self) -> HalfSplitRotation:
        return HalfSplitRotation(self.rope_dim, self.scale, self.theta, self.table)

    def apply(self, qkv, n_heads, n_kv_heads, head_dim, batch) -> None:
        self.runtime.ops.qkv_prepare(
            qkv, n_heads, n_kv_heads, head_dim, batch.positions, batch.slots,
            rope_theta=self.theta, rope_dim=self.rope_dim, rope_scale=self.scale)


class NoPosition(PositionEncoding):
    """Leaves queries and keys as they are."""
    capturable = True


    def apply(self, qkv, n_heads, n_kv_heads, head_dim, batch) -> None:
        return None


register_part("position", "rotary", Rotary)
register_part("position", "none", NoPosition)
