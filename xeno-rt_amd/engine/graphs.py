"""Decode steps as HIP graphs.

A decode step of the Llama-shaped model is several hundred short kernels; launched one
by one, the gaps between them cost as much as the kernels. A step whose sequences all
bring one token has a fixed shape once its batch size and the longest context are
rounded up to buckets, so its kernels are captured once per bucket and replayed with
new contents in the same buffers. Sequences that fill a bucket up are padding (slot -1):
computed, cached nowhere, read by nothing.

All recorded steps take their buffers from one memory pool: the steps are replayed one after
another, never at once, so what one used for its activations serves the next, and only the
inputs and logits of each stay its own. At most MAX_GRAPHS steps are kept; the one replayed
longest ago makes room.
"""
from __future__ import annotations

from typing import Dict, List, Sequence, Tuple

import torch

from ..staging import staging_for
from .batch import StepBatch, pack_step

CONTEXT_BUCKET = 1024    # a recorded step serves contexts up to the next multiple of this (the decode attention cuts its keys by it)
MAX_GRAPHS = 32          # recorded steps kept at a time


def batch_bucket(count: int) -> int:
    """Smallest of 1, 2, 4, 8, 12, 16, 24, 32, 48, 64, 96, 128, ... that holds `count`."""
    power = 1
    while power < count:
        power *= 2
    middle = power // 2 + power // 4          # 1.5 x the power of two below
    return middle if power >= 16 and count <= middle else power


def context_bucket(length: int, limit: int) -> int:
    return min(limit, -(-length // CONTEXT_BUCKET) * CONTEXT_BUCKET)


class DecodeGraph:
    """One captured decode step for `size` sequences whose contexts reach at most `context`."""

    def __init__(self, model, cache, size: int, context: int, device, pool=None):
        self.size = size
        self.context = context
        self.device = device
        # [token ids | positions | slots | sequence slots | offsets | starts | logit rows | rows of the tokens' source]
        self.layout = [size, size, size, size, size + 1, size, size, size]
        total = sum(self.layout)
        self.ints = torch.zeros(total, dtype=torch.int32, device=device)
        cuts, at = [], 0
        for length in self.layout:
            cuts.append(self.ints[at:at + length])
            at += length
        self.batch = StepBatch(
            n_tokens=size, n_sequences=size, token_ids=cuts[0], positions=cuts[1], slots=cuts[2],
            sequence_slots=cuts[3], sequence_offsets=cuts[4], sequence_starts=cuts[5], logit_rows=cuts[6],
            n_logit_rows=size, host_slots=[-1] * size, host_counts=[1] * size, host_starts=[0] * size,
            is_decode=True, max_count=1, max_context=context)
        self.source_rows = cuts[7]
        self.fill([-1] * size, [0] * size, [0] * size)      # all padding: a harmless first run
        # one run outside the graph first: one-time set-up inside kernels' launchers must not be captured
        stream = torch.cuda.Stream(device=device)
        stream.wait_stream(torch.cuda.current_stream(device))
        with torch.cuda.stream(stream):
            model.forward(self.batch, cache)
        torch.cuda.current_stream(device).wait_stream(stream)
        torch.cuda.synchronize(device)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, pool=pool):
            self.logits = model.forward(self.batch, cache)

    def fill(self, slots: Sequence[int], tokens: Sequence[int], starts: Sequence[int], source=None) -> None:
        """New contents for the step's arrays. With source = (tokens on the device, a row for each sequence)
        the token ids are gathered from there, after the upload and before the replay."""
        size, count = self.size, len(slots)
        pad = size - count
        rows = list(source[1]) if source is not None else [0] * count
        # what fills the bucket up are sequences without a slot that bring token 0 at position 0: the host library packs
        # all of them alike, straight into the memory the arrays are uploaded from
        ones = [1] * size
        pack_step(list(slots) + [-1] * pad, ones, list(starts) + [0] * pad, list(tokens) + [0] * pad, ones, [0] * size,
                  self.device, extra=rows + [0] * pad, out=self.ints)
        if source is not None:
            torch.index_select(source[0], 0, self.source_rows[:count], out=self.batch.token_ids[:count])

    def run(self, slots, tokens, starts, source=None) -> torch.Tensor:
        self.fill(slots, tokens, starts, source)
        self.graph.replay()
        return self.logits


class DecodeGraphs:
    def __init__(self, model, cache, device):
        self.model = model
        self.cache = cache
        self.device = device
        self.graphs: Dict[Tuple[int, int], DecodeGraph] = {}       # in the order of their last use
        self.pool = torch.cuda.graph_pool_handle() if torch.device(device).type == "cuda" else None

    def step(self, slots: List[int], tokens: List[int], starts: List[int], source=None) -> torch.Tensor:
        """Logits [len(slots), vocab] of one decode step; a copy, valid until the caller drops it.
        source: (int32 tokens on the device, a row of them for each sequence) instead of `tokens`."""
        size = batch_bucket(len(slots))
        context = context_bucket(max(starts) + 1, self.cache.max_context)
        key = (size, context)
        graph = self.graphs.pop(key, None)
        if graph is None:
            while len(self.graphs) >= MAX_GRAPHS:
                del self.graphs[next(iter(self.graphs))]
            graph = DecodeGraph(self.model, self.cache, size, context, self.device, self.pool)
        self.graphs[key] = graph
        return graph.run(slots, tokens, starts, source)[:len(slots)].clone()
