"""Choosing the next token from logits.

Options and their meaning are the reference's (crates/xrt-runtime/src/sampler.rs):
temperature <= 1e-5 is greedy: the first index of the maximum (:62-65, :83-98);
otherwise the k largest logits are kept (top_k 0 keeps all, :107, :116-145), their
probabilities are softmax((logit - max)/temperature) (:147-164), the shortest
descending prefix whose probability reaches top_p is kept (:166-183), and one
uniform number picks a token by inverse CDF (:185-195). A repetition penalty > 1
divides positive and multiplies negative logits of tokens already in the
sequence, for greedy too (:77-91, :110-125).

The work is done by one kernel on the device for all rows of a batch. Two things
differ from the reference by design: tokens whose logit equals the k-th largest
(or the last of the top_p prefix) are all kept, and the uniform numbers come from
a counter-based generator keyed by (the request's own seed, step), so that a request
draws the same numbers alone and in any batch, whatever its place in it. Requests that
are given one seed therefore draw the same numbers; `request_seed(seed, index)` makes
a seed of its own for each of several prompts that share one.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence

import torch

from ..staging import staging_for

GREEDY_BELOW = 1e-5      # sampler.rs:63


@dataclass(frozen=True)
class SamplerConfig:
    """Defaults are the reference's (sampler.rs:15-25)."""
    temperature: float = 0.8
    top_k: int = 40
    top_p: float = 0.95
    repetition_penalty: float = 1.1
    seed: Optional[int] = None

    def is_greedy(self) -> bool:
        return self.temperature <= GREEDY_BELOW


_MASK = (1 << 64) - 1


def _mix(value: int) -> int:
    """splitmix64 finaliser."""
    value = (value + 0x9E3779B97F4A7C15) & _MASK
    value = ((value ^ (value >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    value = ((value ^ (value >> 27)) * 0x94D049BB133111EB) & _MASK
    return value ^ (value >> 31)


def uniform(seed: int, request: int, step: int) -> float:
    """A number in [0, 1) that depends only on (seed, request, step)."""
    word = _mix(_mix(_mix(seed & _MASK) ^ (request & _MASK)) ^ (step & _MASK))
    return (word >> 40) / float(1 << 24)


def request_seed(seed: int, index: int) -> int:
    """A seed for the index-th of several requests that were given one seed between them."""
    return _mix(_mix(seed & _MASK) ^ ((index + 1) & _MASK)) >> 1


class TokenLog:
    """The tokens of some sequences on the device, for the repetition penalty: what each has when the log is
    made is uploaded once, and the sampling kernel itself appends what it chooses. Without a log the whole
    history of every penalised row goes to the device at every step."""

    def __init__(self, device, sequences: Sequence[Sequence[int]], room: Sequence[int]):
        """room[i]: tokens that sequence i may still get."""
        self.begin: List[int] = []
        at = 0
        for tokens, more in zip(sequences, room):
            self.begin.append(at)
            at += len(tokens) + max(0, int(more))
        host = torch.zeros(max(at, 1), dtype=torch.int32)
        for begin, tokens in zip(self.begin, sequences):
            host[begin:begin + len(tokens)] = torch.tensor(list(tokens), dtype=torch.int32)
        self.end = self.begin[1:] + [at]
        self.tokens = staging_for(device).upload(host)


class Sampler:
    """Samples one token for each row of a batch of logits, on the device."""

    def __init__(self, ops, device):
        self.ops = ops
        self.device = torch.device(device)
        self._last = None           # (what the operands were made from, the operands): a decode loop asks the same again

    def sample(self, logits: torch.Tensor, configs: Sequence[SamplerConfig],
               histories: Sequence[Sequence[int]], draws: Sequence[float], log=None) -> List[int]:
        """The token ids that `launch` chooses, on the host."""
        return self.launch(logits, configs, histories, draws, log).tolist()

    def launch(self, logits: torch.Tensor, configs: Sequence[SamplerConfig],
               histories: Sequence[Sequence[int]], draws: Sequence[float], log=None) -> torch.Tensor:
        """logits [rows, vocab] float32; for each row its options, the tokens of its sequence so
        far (read only if its penalty is > 1) and its uniform number. Returns the token ids as an
        int32 tensor on the device, without waiting for them: a step can be started from them.

        log: (a TokenLog, for each row its sequence's index there). The penalty then reads the tokens
        from the log, of which `histories` only tell the count, and the chosen token is appended."""
        rows = logits.shape[0]
        if logits.dim() != 2 or logits.shape[1] == 0:
            raise ValueError("cannot sample from an empty logits vector")     # sampler.rs:56-60
        if not (rows == len(configs) == len(histories) == len(draws)):
            raise ValueError("one config, history and draw per row of logits")
        history: List[int] = []
        spans: List[int] = []
        append_at: List[int] = []
        for row, (config, tokens) in enumerate(zip(configs, histories)):
            if config.repetition_penalty <= 1.0:
                spans += [0, 0]
                append_at.append(-1)
            elif log is not None:
                begin = log[0].begin[log[1][row]]
                if begin + len(tokens) >= log[0].end[log[1][row]]:
                    raise ValueError(f"row {row}: the log has no room for another token")
                spans += [begin, begin + len(tokens)]
                append_at.append(begin + len(tokens))
            else:
                spans += [len(history), len(history) + len(tokens)]
                history.extend(int(t) for t in tokens)
        # Rows that take the largest logit read no uniform number; when every row does, and nothing is
        # penalised, the operands of the step before serve again and nothing is uploaded.
        greedy = all(c.is_greedy() for c in configs)
        made_from = (tuple(configs), None if greedy else tuple(draws), tuple(history), tuple(spans), log is not None)
        if self._last is not None and self._last[0] == made_from:
            floats, ints = self._last[1]
        else:
            floats = staging_for(self.device).upload(
                [c.temperature for c in configs] + [c.top_p for c in configs]
                + [c.repetition_penalty for c in configs] + [float(d) for d in draws],
                dtype=torch.float32).view(4, rows)
            ints = staging_for(self.device).upload([c.top_k for c in configs] + spans
                                                   + (append_at if log is not None else history))
            self._last = (made_from, (floats, ints))
        out = torch.empty(rows, dtype=torch.int32, device=self.device)
        # rows that the kernels can sample from a few candidates instead of passes over the whole row, and rows
        # that take the largest logit (many workgroups look for it slice by slice, instead of one over the row)
        small_top_k = any(c.is_greedy() or c.top_k <= 64 for c in configs)       # (no top-k is top_k 0: a top-p alone, or a draw from all tokens)
        if log is not None:
            self.ops.sample(logits, out, floats[0], ints[:rows], floats[1], floats[2], log[0].tokens,
                            ints[rows:3 * rows], floats[3], small_top_k=small_top_k, append_at=ints[3 * rows:])
        else:
            self.ops.sample(logits, out, floats[0], ints[:rows], floats[1], floats[2],
                            ints[3 * rows:], ints[rows:3 * rows], floats[3], small_top_k=small_top_k)
        return out
