"""The tokens of one step, as the arrays that parts and kernels read."""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Sequence

import torch

from ..staging import staging_for


@dataclass
class StepBatch:
    """Sequences in the order given; their new tokens packed one after another.

    Device arrays are int32. A token whose slot is negative is padding: it is
    computed but read by nothing, written nowhere and changes no result.
    """
    n_tokens: int                 # packed tokens, padding included
    n_sequences: int
    token_ids: torch.Tensor       # [n_tokens]
    positions: torch.Tensor       # [n_tokens] absolute position of each token in its sequence
    slots: torch.Tensor           # [n_tokens] slot of each token's sequence
    sequence_slots: torch.Tensor  # [n_sequences]
    sequence_offsets: torch.Tensor  # [n_sequences + 1] where each sequence's tokens begin in the packing
    sequence_starts: torch.Tensor   # [n_sequences] tokens the sequence had before this step
    logit_rows: torch.Tensor      # [n_logit_rows] packed indices whose logits are wanted
    n_logit_rows: int
    # the same facts on the host
    host_slots: List[int]
    host_counts: List[int]        # new tokens of each sequence
    host_starts: List[int]
    is_decode: bool               # every sequence brings exactly one token
    max_count: int                # most new tokens of any sequence
    max_context: int              # longest sequence after this step


def build_batch(slots: Sequence[int], tokens: Sequence[Sequence[int]], starts: Sequence[int],
                wants: Sequence[Sequence[int]], device, pad_tokens_to: int = 0) -> StepBatch:
    """Pack the step's sequences. `wants[i]` are indices into `tokens[i]`."""
    token_ids: List[int] = []
    positions: List[int] = []
    token_slots: List[int] = []
    offsets = [0]
    rows: List[int] = []
    for slot, ids, start, want in zip(slots, tokens, starts, wants):
        base = len(token_ids)
        token_ids.extend(int(t) for t in ids)
        positions.extend(range(start, start + len(ids)))
        token_slots.extend([slot] * len(ids))
        offsets.append(len(token_ids))
        rows.extend(base + int(w) for w in want)
    while len(token_ids) < pad_tokens_to:
        token_ids.append(0)
        positions.append(0)
        token_slots.append(-1)
    n_tokens, n_sequences, n_rows = len(token_ids), len(slots), len(rows)
    packed = token_ids + positions + token_slots + list(slots) + offsets + list(starts) + rows
    dev = staging_for(device).upload(packed)
    cuts, at = [], 0
    for size in (n_tokens, n_tokens, n_tokens, n_sequences, n_sequences + 1, n_sequences, n_rows):
        cuts.append(dev[at:at + size])
        at += size
    counts = [len(ids) for ids in tokens]
    return StepBatch(
        n_tokens=n_tokens, n_sequences=n_sequences,
        token_ids=cuts[0], positions=cuts[1], slots=cuts[2], sequence_slots=cuts[3],
        sequence_offsets=cuts[4], sequence_starts=cuts[5], logit_rows=cuts[6], n_logit_rows=n_rows,
        host_slots=list(slots), host_counts=counts, host_starts=list(starts),
        is_decode=all(c == 1 for c in counts), max_count=max(counts),
        max_context=max(s + c for s, c in zip(starts, counts)))
