"""Helpers of the GPU tests: tolerances, schedules, comparison with the plain model."""
import torch

# Largest difference allowed between the engine's logits and the plain implementation's,
# relative to the largest logit of the compared block.
#   float32: both sides round each operation to 2^-24; sums of a few hundred to a few thousand terms in
#            different orders differ by about 1e-6 of the largest term (the kernels add up in two levels,
#            pieces of 8 or 16 terms and then the pieces' sums, which keeps a long sum's rounding small).
#            Largest errors seen over all tests: max 4.2e-6, rms 9.5e-7; the limits are 2.4 and 2.6 times that.
#   bfloat16: activations are rounded to 8 bits (2^-9 relative) about six times per layer;
#            with the tests' weights (std 0.2: sharp attention, gains above one) that comes
#            to one or two percent of the largest logit. The root-mean-square bound is
#            tighter because it does not ride on the single worst element. Largest errors seen over all
#            tests (printed at the end of every run, with the test that had them): max 4.0e-2, rms 7.0e-3 with
#            the tiny models' weights of std 0.2 (the stand-in for the kernels on the CPU, which shares no code
#            with them, has 3.6e-2 at the same request); max 1.5e-2, rms 2.9e-3 at real layer sizes with std 0.02.
TOLERANCE = {"float32": dict(max=1e-5, rms=2.5e-6), "bfloat16": dict(max=5e-2, rms=1.5e-2)}


def errors(got: torch.Tensor, want: torch.Tensor):
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    assert got.shape == want.shape, (got.shape, want.shape)
    scale = float(want.abs().max())
    diff = got - want
    return float(diff.abs().max()) / scale, float(diff.pow(2).mean().sqrt()) / scale


SEEN = {}       # dtype -> [largest max error, largest rms error, what had the former] that passed: printed at the end of a run


def assert_logits(got, want, dtype, what=""):
    assert torch.isfinite(got).all(), f"{what}: logits are not finite"
    worst, rms = errors(got, want)
    seen = SEEN.setdefault(dtype, [0.0, 0.0, ""])
    if worst > seen[0]:
        seen[0], seen[2] = worst, what
    seen[1] = max(seen[1], rms)
    limit = TOLERANCE[dtype]
    assert worst <= limit["max"] and rms <= limit["rms"], \
        f"{what} [{dtype}]: max error {worst:.3e} (limit {limit['max']:.1e}), rms {rms:.3e} (limit {limit['rms']:.1e})"
    return worst, rms


def first_bad_position(got, want, dtype):
    """Index of the first row whose error exceeds the limit, or None: where to look first."""
    limit = TOLERANCE[dtype]["max"]
    scale = float(want.abs().max())
    for t in range(want.shape[0]):
        if float((got[t].double().cpu() - want[t].double()).abs().max()) / scale > limit:
            return t
    return None


def plain_matrix(weight):
    """A bound weight as a matrix with rows contiguous along k, whichever layout the kernels keep it in."""
    return weight.unpacked() if hasattr(weight, "unpacked") else weight


def token_ids(vocab, length, seed):
    return torch.randint(0, vocab, (length,), generator=torch.Generator().manual_seed(seed)).tolist()


def run_whole(engine, ids):
    """One request alone, whole, logits at every position."""
    slot = engine.alloc_slot()
    try:
        return engine.step([(slot, ids, list(range(len(ids))))])
    finally:
        engine.free_slot(slot)


def run_tail_decoded(engine, ids, tail=32):
    """The first len - tail tokens in one step (at least one), the rest one by one."""
    head = max(1, len(ids) - tail)
    slot = engine.alloc_slot()
    try:
        rows = [engine.step([(slot, ids[:head], list(range(head)))])]
        for t in range(head, len(ids)):
            rows.append(engine.step([(slot, [ids[t]], [0])]))
        return torch.cat(rows)
    finally:
        engine.free_slot(slot)


def run_batched(engine, requests, prompts):
    """All requests start together: request i brings its first prompts[i] tokens in one step, then
    one token per step; a request whose tokens are used up ends (its slot is freed) while the
    others go on. Returns the logits [len, vocab] of every request."""
    slots = [engine.alloc_slot() for _ in requests]
    rows = [[] for _ in requests]
    done = [False] * len(requests)
    try:
        logits = engine.step([(slot, ids[:p], list(range(p))) for slot, ids, p in zip(slots, requests, prompts)])
        at = 0
        for i, p in enumerate(prompts):
            rows[i].append(logits[at:at + p]); at += p
        position = list(prompts)
        while True:
            for i, ids in enumerate(requests):
                if not done[i] and position[i] >= len(ids):
                    engine.free_slot(slots[i]); done[i] = True
            live = [i for i in range(len(requests)) if not done[i]]
            if not live:
                break
            logits = engine.step([(slots[i], [requests[i][position[i]]], [0]) for i in live])
            for row, i in enumerate(live):
                rows[i].append(logits[row:row + 1]); position[i] += 1
        return [torch.cat(r) for r in rows]
    finally:
        for i, slot in enumerate(slots):
            if not done[i]:
                engine.free_slot(slot)


def assert_greedy_tokens(logits_of, prompt, tokens, dtype, penalty=1.0, what=""):
    """`tokens` are what greedy generation from `prompt` gives, by the plain logits `logits_of(ids) -> [len, vocab]`:
    in 32-bit every token is the plain loop's choice; in bfloat16 every token is, given the tokens before it, within
    twice the logits' tolerance of the plain model's best (two near-equal logits may change places)."""
    import plain_llama as P
    history = list(prompt)
    for index, token in enumerate(tokens):
        row = P.apply_repetition_penalty(logits_of(history)[-1].float(), history, penalty)
        if dtype == "float32":
            assert token == P.greedy(row), f"{what}: token {index} is {token}, the plain loop chooses {P.greedy(row)}"
        else:
            assert float(row.max() - row[token]) <= 2 * TOLERANCE[dtype]["max"] * float(row.abs().max()), \
                f"{what}: token {index} ({token}) is not among the plain model's best"
        history.append(token)
