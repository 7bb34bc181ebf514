"""The tokens of one step, as the arrays that parts and kernels read."""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import List, Sequence

import numpy as np
import torch

from ..host import StepFacts, last_error, load_host
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


def _int32(values) -> np.ndarray:
    return np.ascontiguousarray(values, dtype=np.int32)


def flatten(lists: Sequence[Sequence[int]]):
    """(the lists' lengths, their members one after another), both int32."""
    counts = _int32([len(members) for members in lists])
    flat = np.concatenate([_int32(members) for members in lists]) if len(lists) else np.zeros(0, dtype=np.int32)
    return counts, _int32(flat)


def pack_step(slots, counts, starts, tokens, want_counts, wants, device, pad_tokens_to: int = 0, extra: Sequence[int] = (),
              out: torch.Tensor = None, allocate=None):
    """The step's arrays, packed by the host library (csrc/host/xrt_host.cpp: xrt_step_pack) straight into the memory
    they are uploaded from: returns (int32 tensor on the device: [token ids | positions | slots | sequence slots |
    offsets | starts | logit rows | extra], the step's facts). All arguments are int32 arrays; tokens and wants are flat."""
    lib = load_host()
    slots, counts, starts, tokens = _int32(slots), _int32(counts), _int32(starts), _int32(tokens)
    want_counts, wants, extra = _int32(want_counts), _int32(wants), _int32(extra)
    n = len(slots)
    room = int(lib.xrt_step_room(n, len(tokens), len(wants), int(pad_tokens_to)))
    facts = StepFacts()
    status = []

    def fill(host: np.ndarray) -> None:
        status.append(lib.xrt_step_pack(n, slots.ctypes.data, counts.ctypes.data, starts.ctypes.data, tokens.ctypes.data,
                                        want_counts.ctypes.data, wants.ctypes.data, int(pad_tokens_to), host.ctypes.data,
                                        room, ctypes.byref(facts)))
        host[room:] = extra

    if out is None and allocate is not None:
        out = allocate(room + len(extra))
    packed = staging_for(device).upload_filled(room + len(extra), fill, out=out)
    if status[0] != 0:
        raise ValueError(last_error())
    return packed, facts


def build_batch(slots: Sequence[int], tokens: Sequence[Sequence[int]], starts: Sequence[int],
                wants: Sequence[Sequence[int]], device, pad_tokens_to: int = 0, allocate=None) -> StepBatch:
    """Pack the step's sequences. `wants[i]` are indices into `tokens[i]`. allocate(count): where the int32 arrays
    lie on the device (None: a tensor of their own)."""
    counts, flat_tokens = flatten(tokens)
    want_counts, flat_wants = flatten(wants)
    dev, facts = pack_step(slots, counts, starts, flat_tokens, want_counts, flat_wants, device, pad_tokens_to, allocate=allocate)
    n_tokens, n_sequences, n_rows = facts.n_tokens, len(slots), facts.n_rows
    cuts, at = [], 0
    for size in (n_tokens, n_tokens, n_tokens, n_sequences, n_sequences + 1, n_sequences, n_rows):
        cuts.append(dev[at:at + size])
        at += size
    return StepBatch(
        n_tokens=n_tokens, n_sequences=n_sequences,
        token_ids=cuts[0], positions=cuts[1], slots=cuts[2], sequence_slots=cuts[3],
        sequence_offsets=cuts[4], sequence_starts=cuts[5], logit_rows=cuts[6], n_logit_rows=n_rows,
        host_slots=[int(s) for s in slots], host_counts=counts.tolist(), host_starts=[int(s) for s in starts],
        is_decode=bool(facts.is_decode), max_count=facts.max_count, max_context=facts.max_context)
