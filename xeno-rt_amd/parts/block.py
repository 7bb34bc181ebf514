"""Pre-norm block: x += mixer(norm1(x)); x += feed_forward(norm2(x)).

The order of the reference's layer loop (crates/xrt-models/src/llama.rs:433-602):
norm, attention, add, norm, feed-forward, add. The residual stream x is float32
and is updated in place; each part adds its own output to it.
"""
from __future__ import annotations

from typing import Dict

from .base import Block, CacheNeeds, Runtime, WeightSpec, register_part


class PreNormBlock(Block):
    def __init__(self, mixer_norm, mixer, feed_forward_norm, feed_forward):
        self.mixer_norm = mixer_norm
        self.mixer = mixer
        self.feed_forward_norm = feed_forward_norm
        self.feed_forward = feed_forward

    def parts(self):
        return (self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward)

    @property
    def capturable(self) -> bool:
        return all(part.capturable for part in self.parts())

    def weight_specs(self) -> Dict[str, WeightSpec]:
        specs: Dict[str, WeightSpec] = {}
        for part in self.parts():
            specs.update(part.weight_specs())
        return specs

    def cache_needs(self) -> CacheNeeds:
        return self.mixer.cache_needs()

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        for part in self.parts():
            part.bind(tensors, runtime)

    @property
    def passes_norms(self) -> bool:
        return bool(getattr(self.mixer, "passes_norms", False))

    def first_norm(self):
        return self.mixer_norm

    def forward(self, x, batch, cache, h=None, then=None):
        if h is None:
            h = self.mixer_norm.forward(x)
        # a norm is left to the products around it only if the part after it reads nothing but products of it
        if self.passes_norms and getattr(self.feed_forward, "passes_norms", False):
            h = self.mixer.forward(h, batch, cache, x, then=self.feed_forward_norm)
        else:
            h = self.mixer.forward(h, batch, cache, x)
        if h is None:
            h = self.feed_forward_norm.forward(x)
        if then is not None and getattr(self.feed_forward, "passes_norms", False):
            return self.feed_forward.forward(h, batch, x, then=then)
        self.feed_forward.forward(h, batch, x)
        return None


register_part("block", "pre_norm", PreNormBlock)
