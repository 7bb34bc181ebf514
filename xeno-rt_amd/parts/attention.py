"""Causal attention with grouped key/value heads over the cache.

The reference's attention (crates/xrt-models/src/llama.rs:447-577 decode,
:695-784 prefill): q, k, v projections without bias; optional RMSNorm of every
head of q and k with one weight [head_dim] each (:1025-1040), after the
projection and before the position encoding; keys (encoded) and values (raw)
appended to the cache; query head h reads key/value head h // group; a token at
position P sees keys 0..P; softmax of q.k * scale in float32; output projection
added to the residual stream.

Q, K and V are bound as one matrix [(n_heads + 2 n_kv_heads) head_dim][hidden], so
one product reads the normed activations once (the reference fuses the three
dispatches, llama.rs:447-464).
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from .base import CacheNeeds, KVSpec, Mixer, PositionEncoding, Runtime, WeightSpec, register_part


class Attention(Mixer):
    passes_norms = True

    @property
    def capturable(self) -> bool:
        return self.position is None or self.position.capturable

    def __init__(self, prefix: str, hidden: int, n_heads: int, n_kv_heads: int, head_dim: int,
                 position: Optional[PositionEncoding] = None, qk_norm: bool = False,
                 qk_norm_eps: float = 0.0, scale: Optional[float] = None,
                 window: Optional[int] = None):
        if n_heads <= 0 or n_kv_heads <= 0 or n_heads % n_kv_heads != 0:
            raise ValueError(f"head counts {n_heads}/{n_kv_heads}: the first must be a multiple of the second")
        if head_dim <= 0 or head_dim % 2 != 0:          # llama.rs:125-128 takes any size; the rotation pairs dims, so an even one
            raise ValueError(f"head_dim {head_dim} must be positive and even")
        self.prefix = prefix
        self.hidden = hidden
        self.n_heads = n_heads
        self.n_kv_heads = n_kv_heads
        self.head_dim = head_dim
        self.position = position
        self.qk_norm = qk_norm
        self.qk_norm_eps = float(qk_norm_eps)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)  # llama.rs:506
        self.window = window
        self.q_width = n_heads * head_dim
        self.kv_width = n_kv_heads * head_dim
        self.w_qkv = None
        self.w_o = None
        self.q_norm = None
        self.k_norm = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p = self.prefix
        specs = {
            p + "q_proj.weight": WeightSpec((self.q_width, self.hidden)),
            p + "k_proj.weight": WeightSpec((self.kv_width, self.hidden)),
            p + "v_proj.weight": WeightSpec((self.kv_width, self.hidden)),
            p + "o_proj.weight": WeightSpec((self.hidden, self.q_width)),
        }
        if self.qk_norm:
            specs[p + "q_norm.weight"] = WeightSpec((self.head_dim,), init="ones", kind="vector")
            specs[p + "k_norm.weight"] = WeightSpec((self.head_dim,), init="ones", kind="vector")
        return specs

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(kv=KVSpec(self.n_kv_heads, self.head_dim, self.window))

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        p = self.prefix
        if self.position is not None:
            self.position.bind(tensors, runtime)
        # q and k heads that a rotation over the whole head turns: their pairs are kept side by side
        rotation = None if self.position is None else self.position.rotation()
        whole = rotation is not None and rotation.rope_dim == self.head_dim
        self.w_qkv = runtime.weight([tensors[p + name] for name in ("q_proj.weight", "k_proj.weight", "v_proj.weight")],
                                    "rotary", head_dim=self.head_dim,
                                    rotated_heads=self.n_heads + self.n_kv_heads if whole else 0)
        self.w_o = runtime.weight(tensors[p + "o_proj.weight"])
        if self.qk_norm:
            self.q_norm = runtime.vector(tensors[p + "q_norm.weight"])
            self.k_norm = runtime.vector(tensors[p + "k_norm.weight"])

    def forward(self, h, batch, cache, residual: torch.Tensor, then=None):
        rt = self.runtime
        ops = rt.ops
        tokens = h.shape[0]
        kv = cache.kv
        qkv = rt.empty((tokens, self.q_width + 2 * self.kv_width))

        dims = (self.n_heads, self.n_kv_heads, self.head_dim)
        write_to = kv if cache.writable else None
        longest_run = int(getattr(batch, "max_count", 0) or 0)      # picks how the values are written; 0: unknown
        rotation = None if self.position is None else self.position.rotation()
        slopes = None if self.position is None else self.position.score_slopes()
        out = rt.empty((tokens, self.q_width))
        # A decode step of a model with head norms: the projection only, and the attention kernel finishes q, k and v
        # itself (norms, rotation, cache write) where it can; without head norms the projection's own kernel does that.
        finishes = getattr(ops, "attention_finishes_qkv", None)
        if (self.qk_norm and write_to is not None and slopes is None and (rotation is not None or self.position is None)
                and finishes is not None and finishes(qkv.dtype, *dims, batch, self.window, 0 if rotation is None else rotation.rope_dim,
                                                       None if rotation is None else rotation.table)):
            ops.linear(h, self.w_qkv, qkv)
            ops.attention(qkv, *dims, kv, batch, out, scale=self.scale,
                          finish=ops.QkvFinish(self.q_norm, self.k_norm, self.qk_norm_eps, None if rotation is None else rotation.table))
            return ops.linear(out, self.w_o, residual, accumulate=True,
                              then_norm=None if then is None else then.row_scale())
        if rotation is not None or self.position is None:
            # the projection, then in one pass (in the same kernel, where a step is short): head norms, rotation, cache write
            ops.linear_qkv(h, self.w_qkv, qkv, *dims, batch.positions, batch.slots,
                            q_norm=self.q_norm, k_norm=self.k_norm, norm_eps=self.qk_norm_eps,
                            rope_theta=None if rotation is None else rotation.theta,
                            rope_dim=0 if rotation is None else rotation.rope_dim,
                            rope_scale=1.0 if rotation is None else rotation.scale,
                            kv=write_to, longest_run=longest_run)
        else:
            # any other position encoding: norms, then the encoding, then the cache write
            ops.linear(h, self.w_qkv, qkv)
            if self.qk_norm:
                ops.qkv_prepare(qkv, *dims, batch.positions, batch.slots,
                                q_norm=self.q_norm, k_norm=self.k_norm, norm_eps=self.qk_norm_eps)
            self.position.apply(qkv, *dims, batch)
            if write_to is not None:
                ops.qkv_prepare(qkv, *dims, batch.positions, batch.slots, kv=write_to, longest_run=longest_run)

        ops.attention(qkv, *dims, kv, batch, out, scale=self.scale, window=self.window,
                      **({} if slopes is None else {"distance_slopes": slopes}))
        return ops.linear(out, self.w_o, residual, accumulate=True,
                          then_norm=None if then is None else then.row_scale())


register_part("mixer", "attention", Attention)
