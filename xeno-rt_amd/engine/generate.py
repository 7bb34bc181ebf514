"""The generation loop above the step function.

For one sequence it is the reference's loop (crates/xrt-runtime/src/session.rs:69-141):
prefill the whole prompt, then repeatedly sample from the last logits; a stop
token ends the request and is neither stored nor returned (:117-119); a full
context ends it (:120-122); otherwise the token is stored, returned and run
(:124-141). Here it runs batches: the prompts of a batch (unequal lengths) go
through one step, then every live sequence brings one token per step; a
sequence that ends leaves the batch and the others go on; when all have ended
their slots are given back and the next batch starts, as often as there are
requests.

The decisions are plain functions of host values, apart from the engine, so
they can be tested without one.
"""
from __future__ import annotations

import ctypes
import random
from dataclasses import dataclass, field
from typing import Callable, List, Optional, Sequence

from ..host import FINISH_REASONS, last_error, load_host
from ..sampling import SamplerConfig, uniform


@dataclass
class GenerateRequest:
    """Defaults are the reference's (session.rs:25-36)."""
    prompt_ids: Sequence[int]
    max_tokens: int = 128
    temperature: float = 0.8
    top_k: int = 40
    top_p: float = 0.95
    repetition_penalty: float = 1.1
    seed: Optional[int] = None
    stop_ids: Optional[Sequence[int]] = None     # None: the configuration's eos token ids

    def sampler_config(self) -> SamplerConfig:
        return SamplerConfig(self.temperature, self.top_k, self.top_p, self.repetition_penalty, self.seed)


@dataclass
class GenerateResult:
    tokens: List[int]
    finish_reason: str          # "stop" (stop token), "length" (max_tokens), "context" (context full)
    prompt_length: int


@dataclass
class _Live:
    index: int                  # position of the request in the caller's list
    slot: int
    request: GenerateRequest
    history: List[int]
    stops: frozenset
    seed: int
    produced: List[int] = field(default_factory=list)
    finish_reason: Optional[str] = None


def resolve_prompt(prompt_ids: Sequence[int], bos_token_id: Optional[int], context: int) -> List[int]:
    """The tokens that are prefilled: an empty prompt becomes [bos] (session.rs:78-86);
    a prompt longer than the context is an error (session.rs:87-93)."""
    tokens = [int(t) for t in prompt_ids]
    if not tokens:
        if bos_token_id is None:
            raise ValueError("empty prompt and the model has no BOS token")
        tokens = [int(bos_token_id)]
    if len(tokens) > context:
        raise ValueError(f"prompt length {len(tokens)} exceeds model context length {context}")
    return tokens


def decide(token: int, stops, history_length: int, context: int, produced: int, max_tokens: int):
    """What happens to a sampled token: (keep it?, finish reason or None).

    Order of the reference's loop body (session.rs:116-124): stop token first, then
    full context, then the token is kept; the loop condition (:115) ends the request
    once max_tokens are kept, which here also spares the forward pass of the last token.
    The decision is the host library's (csrc/host/xrt_host.cpp: xrt_loop_decide).
    """
    stop_array = (ctypes.c_int * max(1, len(stops)))(*sorted(stops))
    keep = ctypes.c_int(0)
    reason = load_host().xrt_loop_decide(int(token), stop_array, len(stops), int(history_length), int(context),
                                         int(produced), int(max_tokens), ctypes.byref(keep))
    return bool(keep.value), FINISH_REASONS[reason]


def goes_on_whatever_it_draws(history_length: int, context: int, produced: int, max_tokens: int) -> bool:
    """Whether only a stop token can end the request at the token being sampled: then its next step may
    start before the token has been looked at. The same conditions as in `decide` and in the loop below."""
    return bool(load_host().xrt_loop_goes_on_whatever_it_draws(int(history_length), int(context), int(produced), int(max_tokens)))


def plan_batches(prompt_lengths: Sequence[int], max_tokens: Sequence[int], batch_size: int,
                 block_tokens: int, cache_tokens: int, context: int) -> List[List[int]]:
    """Cut the requests, in order, into batches that fit the slots and the cache.

    A request may come to hold min(context, prompt + max_tokens) tokens, rounded up to blocks."""
    n = len(prompt_lengths)
    lengths = (ctypes.c_int * max(1, n))(*[int(v) for v in prompt_lengths])
    limits = (ctypes.c_int * max(1, n))(*[int(v) for v in max_tokens])
    batch_of = (ctypes.c_int * max(1, n))()
    count = load_host().xrt_loop_plan_batches(n, lengths, limits, int(batch_size), int(block_tokens), int(cache_tokens),
                                              int(context), batch_of)
    if count < 0:
        raise ValueError(last_error())
    batches: List[List[int]] = [[] for _ in range(count)]
    for index in range(n):
        batches[batch_of[index]].append(index)
    return batches


def generate(engine, requests: Sequence[GenerateRequest], batch_size: Optional[int] = None,
             on_token: Optional[Callable[[int, int], None]] = None, sampler=None) -> List[GenerateResult]:
    """Generate for every request; results in the order of the requests.

    on_token(request_index, token_id) is called for every token kept, as it is produced.
    """
    from ..cache import BLOCK_TOKENS
    from ..sampling import TokenLog
    from ..staging import staging_for

    config = engine.config
    context = engine.max_context
    if sampler is None:
        from ..sampling import Sampler
        sampler = Sampler(engine.ops, engine.device)
    default_stops = tuple(getattr(config, "eos_token_ids", ()) or ())
    bos = getattr(config, "bos_token_id", None)
    prompts = [resolve_prompt(r.prompt_ids, bos, context) for r in requests]
    if batch_size is None:
        batch_size = engine.cache.max_slots
    batch_size = max(1, min(batch_size, engine.cache.max_slots))
    batches = plan_batches([len(p) for p in prompts], [r.max_tokens for r in requests], batch_size,
                           BLOCK_TOKENS, engine.cache.n_blocks * BLOCK_TOKENS, context)
    results: List[Optional[GenerateResult]] = [None] * len(requests)

    for batch in batches:
        live: List[_Live] = []
        try:
            for index in batch:
                request = requests[index]
                stops = frozenset(default_stops if request.stop_ids is None else request.stop_ids)
                seed = request.seed if request.seed is not None else random.getrandbits(63)  # sampler.rs:37
                live.append(_Live(index, engine.alloc_slot(), request, list(prompts[index]), stops, seed))
            done = [seq for seq in live if seq.request.max_tokens <= 0]
            for seq in done:
                seq.finish_reason = "length"
            running = [seq for seq in live if seq.finish_reason is None]
            if running:
                logits = engine.step([(seq.slot, seq.history, [len(seq.history) - 1]) for seq in running])
            # One step ahead of the host: the next step starts from the sampled tokens on the device, for
            # every request that only a stop token could end, and the host looks at the tokens while it
            # runs. A request that did draw a stop token has then been stepped once for nothing; its row
            # of logits is dropped. The tokens that a repetition penalty reads are kept on the device.
            log, place = None, {}
            if any(seq.request.repetition_penalty > 1.0 for seq in running):
                log = TokenLog(engine.device, [seq.history for seq in running],
                               [min(seq.request.max_tokens, context - len(seq.history)) + 1 for seq in running])
                place = {seq.index: at for at, seq in enumerate(running)}
            while running:
                drawn = sampler.launch(
                    logits, [seq.request.sampler_config() for seq in running],
                    [seq.history for seq in running],
                    [uniform(seq.seed, 0, len(seq.produced)) for seq in running],
                    log=None if log is None else (log, [place[seq.index] for seq in running]))
                fetched = staging_for(engine.device).fetch(drawn)
                stepped = [(row, seq) for row, seq in enumerate(running)
                           if goes_on_whatever_it_draws(len(seq.history), context, len(seq.produced),
                                                        seq.request.max_tokens)]
                if stepped:
                    logits = engine.step_from(drawn, [(seq.slot, row) for row, seq in stepped])
                still = []
                for seq, token in zip(running, fetched.values()):
                    keep, reason = decide(token, seq.stops, len(seq.history), context,
                                          len(seq.produced), seq.request.max_tokens)
                    if keep:
                        seq.history.append(token)
                        seq.produced.append(token)
                        if on_token is not None:
                            on_token(seq.index, token)
                    if reason is None and len(seq.history) >= context:
                        reason = "context"      # the next token would find the context full
                    seq.finish_reason = reason
                    if reason is None:
                        still.append(seq)
                kept = [i for i, (_, seq) in enumerate(stepped) if seq.finish_reason is None]
                if [stepped[i][1] for i in kept] != still:
                    raise RuntimeError("a request went on that was not stepped ahead")
                if still and len(kept) < len(stepped):
                    logits = logits.index_select(0, staging_for(engine.device).upload(kept))
                running = still
        finally:
            for seq in live:
                engine.free_slot(seq.slot)
        for seq in live:
            results[seq.index] = GenerateResult(seq.produced, seq.finish_reason, len(prompts[seq.index]))
    return results
