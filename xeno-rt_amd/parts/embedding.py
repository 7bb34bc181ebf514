"""Token embedding and output head.

Embedding: x = E[token_id, :], no scaling (crates/xrt-models/src/llama.rs:1042-1055).
Head: logits = W y in float32, W = lm_head.weight, or the embedding table when
the model ties them (llama.rs:299-305, 604-613).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import Part, Runtime, WeightSpec


class Embedding(Part):
    capturable = True

    def __init__(self, prefix: str, vocab: int, hidden: int):
        self.prefix = prefix
        self.vocab = vocab
        self.hidden = hidden
        self.table = None
        self.shared_with_head = False       # set by an OutputHead that is tied to this table

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {self.prefix + "weight": WeightSpec((self.vocab, self.hidden))}

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        # a table that is also the head's weight is kept as products like it; one that is only looked up stays plain
        tensor = tensors[self.prefix + "weight"]
        self.table = runtime.weight(tensor) if self.shared_with_head else runtime.matrix(tensor)

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        """float32 residual stream [tokens, hidden] for int32 token ids."""
        x = self.runtime.empty((token_ids.shape[0], self.hidden), torch.float32)
        self.runtime.ops.embed(self.table, token_ids, x)
        return x


class OutputHead(Part):
    capturable = True

    def __init__(self, prefix: str, vocab: int, hidden: int, tied_to: Optional[Embedding] = None):
        self.prefix = prefix
        self.vocab = vocab
        self.hidden = hidden
        self.tied_to = tied_to
        if tied_to is not None:
            tied_to.shared_with_head = True
        self.weight = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        if self.tied_to is not None:
            return {}
        return {self.prefix + "weight": WeightSpec((self.vocab, self.hidden))}

    def ignored_names(self):
        """Tensors that a checkpoint may carry and that this part does not read."""
        return [self.prefix + "weight"] if self.tied_to is not None else []

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        if self.tied_to is not None:
            self.weight = self.tied_to.table        # the same buffer, not a copy
        else:
            self.weight = runtime.weight(tensors[self.prefix + "weight"])

    def forward(self, y: torch.Tensor) -> torch.Tensor:
        logits = self.runtime.empty((y.shape[0], self.vocab), torch.float32, outlives_the_step=True)
        self.runtime.ops.linear(y, self.weight, logits)
        return logits
