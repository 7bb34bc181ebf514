"""The decoder that every architecture is an instance of: embedding, a schedule
of layer calls, final norm, output head.

The schedule is a list. An entry names a layer and may name it again (the same
weights run twice, each call with a cache entry of its own), or may read the
cache entry of an earlier call instead of owning one.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from ..parts.base import Block, CacheNeeds, Norm, Runtime, WeightSpec
from ..parts.embedding import Embedding, OutputHead


@dataclass(frozen=True)
class LayerCall:
    """One entry of the schedule: run `layer`; keep its keys/values/state in the
    cache entry of this call, or read (not write) the entry of call `reads_cache_of`."""
    layer: int
    reads_cache_of: Optional[int] = None


@dataclass
class ModelSpec:
    config: object
    embedding: Embedding
    layers: List[Block]
    final_norm: Norm
    head: OutputHead
    schedule: Optional[List[LayerCall]] = None

    def __post_init__(self):
        if self.schedule is None:
            self.schedule = [LayerCall(i) for i in range(len(self.layers))]
        for index, call in enumerate(self.schedule):
            if not 0 <= call.layer < len(self.layers):
                raise ValueError(f"schedule entry {index} names layer {call.layer} of {len(self.layers)}")
            if call.reads_cache_of is not None:
                source = call.reads_cache_of
                if not 0 <= source < index:
                    raise ValueError(f"schedule entry {index} reads the cache of entry {source}, "
                                     "which must be an earlier entry")
                if self.schedule[source].reads_cache_of is not None:
                    raise ValueError(f"schedule entry {index} reads the cache of entry {source}, "
                                     "which owns none")
                if (self.layers[call.layer].cache_needs()
                        != self.layers[self.schedule[source].layer].cache_needs()):
                    raise ValueError(f"schedule entry {index} reads the cache of entry {source}, "
                                     "whose layer keeps something else")

    def parts(self):
        return [self.embedding, *self.layers, self.final_norm, self.head]

    def weight_specs(self) -> Dict[str, WeightSpec]:
        specs: Dict[str, WeightSpec] = {}
        for part in self.parts():
            for name, spec in part.weight_specs().items():
                if name in specs and specs[name] != spec:
                    raise ValueError(f"tensor {name} is declared twice with different shapes")
                specs[name] = spec
        return specs

    def capturable(self) -> bool:
        """Whether a decode step of this model can be recorded as a graph and replayed."""
        return all(part.capturable for part in self.parts())

    def ignored_names(self) -> List[str]:
        return list(self.head.ignored_names())

    def cache_needs(self) -> List[Optional[CacheNeeds]]:
        """For each schedule entry what its cache entry holds, None if it reads another's."""
        return [None if call.reads_cache_of is not None else self.layers[call.layer].cache_needs()
                for call in self.schedule]


class DecoderModel:
    """A ModelSpec with its weights bound: runs the tokens of one step."""

    def __init__(self, spec: ModelSpec, tensors: Dict[str, torch.Tensor], runtime: Runtime):
        self.spec = spec
        self.config = spec.config
        self.runtime = runtime
        for part in spec.parts():
            part.bind(tensors, runtime)

    def forward(self, batch, cache) -> torch.Tensor:
        """Logits [len(batch.logit_rows), vocab] in float32 for the tokens of `batch`."""
        spec = self.spec
        x = spec.embedding.forward(batch.token_ids)
        h = None            # the next block's first norm of x, where the block before it has made it already
        for index, call in enumerate(spec.schedule):
            block = spec.layers[call.layer]
            if not getattr(block, "passes_norms", False):
                block.forward(x, batch, cache.layer_cache(index))
                h = None
                continue
            after = spec.layers[spec.schedule[index + 1].layer] if index + 1 < len(spec.schedule) else None
            then = after.first_norm() if after is not None and getattr(after, "passes_norms", False) else None
            h = block.forward(x, batch, cache.layer_cache(index), h=h, then=then)
        if batch.n_logit_rows == 0:
            return self.runtime.empty((0, spec.head.vocab), torch.float32, outlives_the_step=True)
        y = spec.final_norm.forward(x, rows=batch.logit_rows)
        return spec.head.forward(y)
