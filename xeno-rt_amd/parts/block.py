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

    def forward(self, x, batch, cache) -> None:
        h = self.mixer_norm.forward(x)
        self.mixer.forward(h, batch, cache, x)
        h = self.feed_forward_norm.forward(x)
        self.feed_forward.forward(h, batch, x)


register_part("block", "pre_norm", PreNormBlock)
