"""The generation loop's decisions and the step function's checks, on the CPU: the
engine's own step function, cache and loop run with the test stand-in for the kernels."""
import pytest
import torch

from conftest import TINY, make_folder
from ops_emulation import EmulatedOps
import plain_llama as P
from xeno_rt_amd.engine import (Engine, GenerateRequest, StepError, decide, generate, plan_batches,
                                resolve_prompt)
from xeno_rt_amd.engine.generate import goes_on_whatever_it_draws
from xeno_rt_amd.sampling import Sampler, SamplerConfig, TokenLog, uniform

GREEDY = dict(temperature=0.0, repetition_penalty=1.0)


@pytest.fixture(scope="module")
def pair(tmp_path_factory):
    folder = make_folder(TINY["llama"], tmp_path_factory.mktemp("loop"), seed=4, std=0.2)
    engine = Engine.load(folder, dtype="float32", device="cpu", ops=EmulatedOps(), max_tokens=64 * 6, max_slots=3)
    return engine, P.PlainModel(folder)


def test_decide_follows_the_references_order():
    stops = {1}
    assert decide(1, stops, 5, 10, 0, 4) == (False, "stop")          # session.rs:117-119, checked first
    assert decide(7, stops, 10, 10, 0, 4) == (False, "context")      # session.rs:120-122
    assert decide(1, stops, 10, 10, 0, 4) == (False, "stop")
    assert decide(7, stops, 5, 10, 0, 4) == (True, None)
    assert decide(7, stops, 5, 10, 3, 4) == (True, "length")         # the last allowed token is kept
    assert decide(7, set(), 5, 10, 0, 1) == (True, "length")


def test_resolve_prompt():
    assert resolve_prompt([], 3, 10) == [3]                          # session.rs:78-86
    with pytest.raises(ValueError, match="no BOS"):
        resolve_prompt([], None, 10)
    with pytest.raises(ValueError, match="exceeds model context length"):
        resolve_prompt(list(range(11)), 0, 10)                       # session.rs:87-93
    assert resolve_prompt(list(range(10)), 0, 10) == list(range(10))


def test_plan_batches_respects_slots_and_cache():
    assert plan_batches([5, 5, 5, 5, 5], [10] * 5, 2, 64, 64 * 100, 128) == [[0, 1], [2, 3], [4]]
    # 60 + 10 tokens round up to 128 each: two fit into 256, not three
    assert plan_batches([60, 60, 60], [10, 10, 10], 8, 64, 256, 128) == [[0, 1], [2]]
    # the context bounds what a request can come to hold
    assert plan_batches([60, 60], [1000, 1000], 8, 64, 256, 128) == [[0, 1]]
    with pytest.raises(ValueError, match="may hold"):
        plan_batches([300], [10], 8, 64, 256, 512)


def test_uniform_depends_on_seed_and_step_only():
    draws = [uniform(5, 0, step) for step in range(200)]
    assert all(0.0 <= d < 1.0 for d in draws) and len(set(draws)) > 190
    assert draws[:3] == [uniform(5, 0, 0), uniform(5, 0, 1), uniform(5, 0, 2)]
    assert uniform(6, 0, 0) != draws[0]
    assert 0.4 < sum(draws) / len(draws) < 0.6


def test_batches_of_unequal_prompts_match_the_plain_loop(pair):
    engine, plain = pair
    prompts = [[4, 8, 15, 16, 23], [42], list(range(30, 47)), [9, 9, 9], [7] * 11, [200, 100]]
    limits = [6, 9, 3, 1, 5, 7]
    requests = [GenerateRequest(p, max_tokens=n, stop_ids=[], **GREEDY) for p, n in zip(prompts, limits)]
    seen = []
    results = generate(engine, requests, batch_size=3, on_token=lambda i, t: seen.append((i, t)))
    for prompt, limit, result in zip(prompts, limits, results):
        assert result.tokens == P.generate_greedy(plain, prompt, limit, stop_ids=[])
        assert result.finish_reason == "length" and result.prompt_length == len(prompt)
    for index, result in enumerate(results):
        assert [t for i, t in seen if i == index] == result.tokens
    engine.cache.check()
    assert engine.cache.slots.n_held == 0 and engine.cache.held_blocks() == 0   # two batches, slots used again


def test_stop_tokens_end_a_request_early_and_are_not_returned(pair):
    engine, plain = pair
    prompt = [4, 8, 15]
    free = P.generate_greedy(plain, prompt, 8, stop_ids=[])
    stop = free[3]
    other = [50, 60]
    results = generate(engine, [GenerateRequest(prompt, max_tokens=8, stop_ids=[stop], **GREEDY),
                                GenerateRequest(other, max_tokens=8, stop_ids=[], **GREEDY)])
    assert results[0].tokens == free[:free.index(stop)] and results[0].finish_reason == "stop"
    assert results[1].tokens == P.generate_greedy(plain, other, 8, stop_ids=[])   # the longer one went on alone
    # the configuration's eos ids are the default stop set
    default = generate(engine, [GenerateRequest(prompt, max_tokens=8, **GREEDY)])[0]
    assert default.tokens == P.generate_greedy(plain, prompt, 8)


def test_which_requests_may_be_stepped_before_their_token_is_seen():
    """Exactly those that `decide` and the full context let go on with any token that is no stop token."""
    for context in (4, 9):
        for history in range(1, context + 1):
            for max_tokens in (1, 2, 5):
                for produced in range(max_tokens):
                    keep, reason = decide(7, {1}, history, context, produced, max_tokens)
                    goes_on = keep and reason is None and history + 1 < context
                    assert goes_on_whatever_it_draws(history, context, produced, max_tokens) == goes_on


def test_a_step_from_tokens_on_the_device_is_the_step_from_the_same_tokens(pair):
    engine, _ = pair
    prompts = [[4, 8, 15, 16], [42], [7] * 9]

    def run(ahead):
        slots = [engine.alloc_slot() for _ in prompts]
        try:
            engine.step([(slot, ids, []) for slot, ids in zip(slots, prompts)])
            nexts = [11, 250, 3]
            if ahead:       # rows in another order than the sequences, and one row that nobody reads
                drawn = torch.tensor([nexts[2], 99, nexts[0], nexts[1]], dtype=torch.int32)
                first = engine.step_from(drawn, [(slots[0], 2), (slots[1], 3), (slots[2], 0)])
                second = engine.step_from(drawn, [(slots[2], 1)])
            else:
                first = engine.step([(slot, [token], [0]) for slot, token in zip(slots, nexts)])
                second = engine.step([(slots[2], [99], [0])])
            assert [engine.length(slot) for slot in slots] == [5, 2, 11]
            return first.clone(), second.clone()
        finally:
            for slot in slots:
                engine.free_slot(slot)

    for got, want in zip(run(True), run(False)):
        assert torch.equal(got, want)
    slot = engine.alloc_slot()
    try:
        engine.step([(slot, [1, 2], [])])
        with pytest.raises(StepError, match="outside the 2 tokens"):
            engine.step_from(torch.tensor([1, 2], dtype=torch.int32), [(slot, 2)])
        assert engine.length(slot) == 2
    finally:
        engine.free_slot(slot)
    engine.cache.check()


def test_the_loop_runs_a_step_ahead_of_the_host(pair, monkeypatch):
    engine, plain = pair
    calls = {"step": 0, "step_from": 0}
    step, step_from = engine.step, engine.step_from
    monkeypatch.setattr(engine, "step", lambda *a, **k: (calls.__setitem__("step", calls["step"] + 1), step(*a, **k))[1])
    monkeypatch.setattr(engine, "step_from",
                        lambda *a, **k: (calls.__setitem__("step_from", calls["step_from"] + 1), step_from(*a, **k))[1])
    prompt = [4, 8, 15]
    free = P.generate_greedy(plain, prompt, 8, stop_ids=[])
    stop = free[3]
    requests = [GenerateRequest(prompt, max_tokens=8, stop_ids=[stop], **GREEDY),
                GenerateRequest([50, 60], max_tokens=6, stop_ids=[], **GREEDY)]
    results = generate(engine, requests)
    assert results[0].tokens == free[:3] and results[0].finish_reason == "stop"
    assert results[1].tokens == P.generate_greedy(plain, [50, 60], 6, stop_ids=[])
    # the prompts' step, then five steps for six tokens, none of them through the host
    assert calls == {"step": 1, "step_from": 5}
    # with a repetition penalty too: the tokens it reads are kept on the device (the sampler appends them), and
    # they are those that a loop through the host hands to the sampler at every step
    calls.update(step=0, step_from=0)
    # a prompt after which the model, left alone, repeats its second token
    prompt = next(p for p in ([a, a + 1, a + 2] for a in range(3, 250))
                  if (lambda free: free[1] == free[2] and free[0] != free[1])(P.generate_greedy(plain, p, 3, stop_ids=[])))
    penalised = GenerateRequest(prompt, max_tokens=5, stop_ids=[], temperature=0.0, repetition_penalty=3.0)
    got = generate(engine, [penalised, GenerateRequest([50, 60], max_tokens=3, stop_ids=[], **GREEDY)])
    assert calls == {"step": 1, "step_from": 4}
    sampler, slot, history = Sampler(engine.ops, engine.device), engine.alloc_slot(), list(prompt)
    monkeypatch.undo()
    logits = engine.step([(slot, history, [len(history) - 1])])
    for _ in range(5):
        history += sampler.sample(logits, [penalised.sampler_config()], [history], [0.0])
        logits = engine.step([(slot, history[-1:], [0])])
    engine.free_slot(slot)
    assert got[0].tokens == history[len(prompt):]
    free = P.generate_greedy(plain, prompt, 5, stop_ids=[])
    assert free[1] == free[2] and got[0].tokens[:2] == free[:2] and got[0].tokens[2] != free[2]   # a token it chose itself is penalised
    assert got[1].tokens == P.generate_greedy(plain, [50, 60], 3, stop_ids=[])
    engine.cache.check()
    assert engine.cache.slots.n_held == 0 and engine.cache.held_blocks() == 0


def test_context_and_zero_length_limits(pair):
    engine, plain = pair
    context = engine.max_context
    assert context == 128
    prompt = list(range(1, context - 1))                             # two tokens fit
    result = generate(engine, [GenerateRequest(prompt, max_tokens=10, stop_ids=[], **GREEDY)])[0]
    assert result.finish_reason == "context" and len(result.tokens) == 2
    assert result.tokens == P.generate_greedy(plain, prompt, 10, stop_ids=[])
    full = generate(engine, [GenerateRequest(list(range(context)), max_tokens=3, stop_ids=[], **GREEDY)])[0]
    assert full.tokens == [] and full.finish_reason == "context"
    none = generate(engine, [GenerateRequest([1, 2], max_tokens=0, **GREEDY)])[0]
    assert none.tokens == [] and none.finish_reason == "length"
    empty = generate(engine, [GenerateRequest([], max_tokens=2, stop_ids=[], **GREEDY)])[0]
    assert empty.prompt_length == 1 and empty.tokens == P.generate_greedy(plain, [], 2, stop_ids=[])
    with pytest.raises(ValueError, match="exceeds model context length"):
        generate(engine, [GenerateRequest(list(range(context + 1)), max_tokens=1)])
    engine.cache.check()
    assert engine.cache.slots.n_held == 0


def test_sampling_is_the_same_alone_and_in_a_batch(pair):
    engine, _ = pair
    make = lambda seed, prompt: GenerateRequest(prompt, max_tokens=8, temperature=0.9, top_k=20, top_p=0.9,
                                                repetition_penalty=1.3, seed=seed, stop_ids=[])
    together = generate(engine, [make(1, [3, 4, 5]), make(2, [6]), make(1, [3, 4, 5])])
    alone = generate(engine, [make(1, [3, 4, 5])])[0]
    assert together[0].tokens == alone.tokens == together[2].tokens
    assert together[1].tokens != alone.tokens
    assert generate(engine, [make(9, [3, 4, 5])])[0].tokens != alone.tokens


def test_steps_that_cannot_run_are_refused_and_change_nothing(pair):
    engine, plain = pair
    slot = engine.alloc_slot()
    engine.step([(slot, [1, 2, 3], [])])
    held = engine.cache.held_blocks()
    for entries, text in [
        ([], "at least one sequence"),
        ([(slot, [], [])], "at least one token"),                         # llama.rs:624-626
        ([(slot, [256], [0])], "exceeds embedding rows"),                 # llama.rs:1044-1049
        ([(slot, [-1], [0])], "exceeds embedding rows"),
        ([(slot, [1], [1])], "wanted index"),
        ([(2, [1], [0])], "not allocated"),
        ([(slot, [1], [0]), (slot, [2], [0])], "appears twice"),
        ([(slot, [1] * 126, [0])], "context limit"),
    ]:
        with pytest.raises(StepError, match=text):
            engine.step(entries)
        assert engine.length(slot) == 3 and engine.cache.held_blocks() == held
    engine.cache.check()
    # the refused steps left the sequence intact: its next logits are those of the plain model
    fresh = engine.alloc_slot()
    got = engine.step([(fresh, [1, 2, 3, 9], [3])])
    assert float((got[0] - plain.logits([1, 2, 3, 9])[3]).abs().max()) < 1e-4
    engine.free_slot(fresh); engine.free_slot(slot)
    assert engine.cache.held_blocks() == 0


def test_a_step_that_the_cache_cannot_hold_takes_nothing(tmp_path):
    folder = make_folder(TINY["qwen3"], tmp_path / "m", seed=4, std=0.2)
    engine = Engine.load(folder, dtype="float32", device="cpu", ops=EmulatedOps(), max_tokens=128, max_slots=2)
    a, b = engine.alloc_slot(), engine.alloc_slot()
    engine.step([(a, [1, 2, 3], [])])
    with pytest.raises(StepError, match="cannot hold"):
        engine.step([(a, [1] * 70, []), (b, [1] * 10, [])])          # 2 + 1 blocks of 2
    assert engine.cache.held_blocks() == 1 and engine.length(a) == 3 and engine.length(b) == 0
    engine.cache.check()
    engine.step([(b, [1] * 10, [])])                                  # what fits still runs
    assert engine.cache.held_blocks() == 2


def test_padding_changes_no_result(pair):
    from xeno_rt_amd.engine.batch import build_batch
    engine, plain = pair
    slot = engine.alloc_slot()
    ids = [5, 6, 7, 8, 9]
    engine.cache.reserve(slot, 5); engine.cache.sync()
    batch = build_batch([slot], [ids], [0], [[4]], "cpu", pad_tokens_to=16)
    assert batch.n_tokens == 16 and int(batch.slots[5]) == -1
    logits = engine.model.forward(batch, engine.cache)
    engine.cache.commit(slot, 5)
    assert float((logits[0] - plain.logits(ids)[4]).abs().max()) < 1e-4
    nxt = engine.step([(slot, [11], [0])])
    assert float((nxt[0] - plain.logits(ids + [11])[5]).abs().max()) < 1e-4
    engine.free_slot(slot)


def test_command_line_options_are_the_references():
    # crates/xrt-cli/src/main.rs:28-49: names and defaults
    from xeno_rt_amd.cli import build_parser, parse_prompts
    args = build_parser().parse_args(["generate", "--model", "m", "--prompt-ids", "1,2,3"])
    assert (args.max_tokens, args.temperature, args.top_k, args.top_p, args.repetition_penalty, args.seed) == \
        (128, 0.8, 40, 0.95, 1.1, None)
    args = build_parser().parse_args(["generate", "--model", "m", "--prompt-ids", "1 2;3", "--prompt-ids", "",
                                      "--max-tokens", "5", "--temperature", "0", "--top-k", "3", "--top-p", "0.5",
                                      "--repetition-penalty", "1.0", "--seed", "9"])
    assert parse_prompts(args.prompt_ids) == [[1, 2], [3], []]
    assert (args.max_tokens, args.temperature, args.top_k, args.top_p, args.repetition_penalty, args.seed) == \
        (5, 0.0, 3, 0.5, 1.0, 9)
    with pytest.raises(SystemExit):
        build_parser().parse_args(["generate", "--prompt-ids", "1"])          # a model is required


def test_request_defaults_are_the_references():
    # crates/xrt-runtime/src/session.rs:25-36 and sampler.rs:15-25
    request = GenerateRequest([1])
    assert (request.max_tokens, request.temperature, request.top_k, request.top_p, request.repetition_penalty,
            request.seed) == (128, 0.8, 40, 0.95, 1.1, None)
    assert SamplerConfig() == SamplerConfig(0.8, 40, 0.95, 1.1, None)
    assert SamplerConfig(temperature=1e-5).is_greedy() and not SamplerConfig(temperature=2e-5).is_greedy()


def test_python_entry_point_on_the_cpu_stand_in(pair):
    from xeno_rt_amd import Runtime
    engine, plain = pair
    session = Runtime(engine).new_session()
    request = GenerateRequest([4, 8, 15], max_tokens=5, stop_ids=[], **GREEDY)
    want = P.generate_greedy(plain, [4, 8, 15], 5, stop_ids=[])
    assert session.generate(request) == want
    seen = []
    assert session.generate_stream(request, seen.append).tokens == want and seen == want
    session.reset()


def test_engine_conveniences(pair):
    engine, plain = pair
    prompts = [[4, 8, 15], [42, 7]]
    got = engine.generate(prompts, max_tokens=4, stop_ids=[])           # greedy unless told otherwise
    assert got == [P.generate_greedy(plain, p, 4, stop_ids=[]) for p in prompts]
    table = engine.get_tensor("model.embed_tokens.weight")
    assert table.device.type == "cpu" and tuple(table.shape) == (engine.config.vocab_size, engine.config.hidden_size)
    with pytest.raises(KeyError):
        engine.get_tensor("model.no_such.weight")


def test_prompts_that_share_a_seed_draw_from_streams_of_their_own(pair):
    """Engine.generate gives every prompt a seed made from the one it was given and the prompt's index: equal prompts
    sampled with a temperature part ways, the same call gives the same tokens again, and a prompt's tokens do not
    depend on what else is in the call."""
    from xeno_rt_amd.engine import GenerateRequest, generate
    from xeno_rt_amd.sampling import request_seed
    engine, _ = pair
    prompt = [4, 8, 15, 16]
    options = dict(max_tokens=12, temperature=1.5, stop_ids=[])
    first = engine.generate([prompt, prompt, prompt], seed=7, **options)
    assert first[0] != first[1] and first[1] != first[2] and first[0] != first[2]
    assert engine.generate([prompt, prompt, prompt], seed=7, **options) == first
    assert engine.generate([prompt, prompt], seed=8, **options)[0] != first[0]
    alone = generate(engine, [GenerateRequest(prompt, seed=request_seed(7, 1), repetition_penalty=1.0, top_k=0, top_p=1.0, **options)])
    assert alone[0].tokens == first[1]
    assert len({request_seed(7, i) for i in range(1000)} | {request_seed(8, i) for i in range(1000)}) == 2000


def test_norms_are_handed_to_the_products_only_where_every_part_agrees(pair, tmp_path):
    """A norm between two products may be done by them (parts with `passes_norms`); the result is the same
    with and without, and a part that does not say so is never given anything but tensors."""
    from xeno_rt_amd.parts.base import FeedForward

    engine, plain = pair
    ids = [5, 9, 2, 7, 11, 3]
    want = engine.step([(engine.alloc_slot(), ids, list(range(len(ids))))])
    engine.free_slot(0)

    handed = []
    ops = EmulatedOps()
    plain_linear = ops.linear

    def watching_linear(a, w, out, accumulate=False, then_norm=None):
        handed.append((isinstance(a, EmulatedOps.Prescaled), then_norm is not None))
        return plain_linear(a, w, out, accumulate=accumulate, then_norm=then_norm)

    ops.linear = watching_linear
    folder = make_folder(TINY["llama"], tmp_path, seed=4, std=0.2)
    watched = Engine.load(folder, dtype="float32", device="cpu", ops=ops, max_tokens=64 * 6, max_slots=3)
    got = watched.step([(watched.alloc_slot(), ids, list(range(len(ids))))])
    assert torch.allclose(got, want, rtol=0, atol=1e-5 * float(want.abs().max()))
    layers = len(watched.model.spec.layers)
    # per layer: o is followed by the feed-forward's norm, down by the next layer's first norm (the last by none)
    assert sum(1 for _, then in handed if then) == 2 * layers - 1
    # every layer but the first takes its q/k/v projection's rows from the layer before (gate/up, which takes them
    # from o, goes through linear_glu); the output head takes a tensor
    assert sum(1 for scaled, _ in handed if scaled) == layers - 1

    # a feed-forward that does not promise: it is called without `then`, gets a tensor, and the block runs both norms
    class Opaque(FeedForward):
        capturable = True

        def __init__(self, inner):
            self.inner = inner

        def weight_specs(self):
            return self.inner.weight_specs()

        def bind(self, tensors, runtime):
            self.inner.bind(tensors, runtime)

        def forward(self, h, batch, residual):
            assert isinstance(h, torch.Tensor)
            self.inner.forward(h, batch, residual)

    watched.free_slot(0)
    block = watched.model.spec.layers[0]
    block.feed_forward = Opaque(block.feed_forward)
    handed.clear()
    again = watched.step([(watched.alloc_slot(), ids, list(range(len(ids))))])
    assert torch.allclose(again, want, rtol=0, atol=1e-5 * float(want.abs().max()))
    # layer 0's o is no longer followed by a handed norm, and nothing is handed on behind its down
    assert sum(1 for _, then in handed if then) == 2 * layers - 1 - 2
    assert sum(1 for scaled, _ in handed if scaled) == layers - 2


def test_buckets_of_recorded_decode_steps():
    from xeno_rt_amd.engine.graphs import batch_bucket, context_bucket
    sizes = [batch_bucket(n) for n in range(1, 130)]
    assert all(size >= n for n, size in enumerate(sizes, start=1))            # a bucket holds its batch
    assert sizes == sorted(sizes)
    assert sorted(set(sizes)) == [1, 2, 4, 8, 12, 16, 24, 32, 48, 64, 96, 128, 192]
    assert [context_bucket(n, 5000) for n in (1, 1024, 1025, 4096, 4097, 5000)] == [1024, 1024, 2048, 4096, 5000, 5000]


def test_staging_on_the_host_stand_in():
    """Without a GPU the staging area hands the values through: copies, never views of what it was given."""
    from xeno_rt_amd.staging import staging_for
    staging = staging_for("cpu")
    assert staging.upload([3, 1, 2]).tolist() == [3, 1, 2]
    assert staging.upload([0.5, 2.0], dtype=torch.float32).dtype == torch.float32
    table = torch.arange(6, dtype=torch.int32).view(2, 3)
    copy = staging.upload(table[1:2])
    table[1, 0] = 99
    assert copy.tolist() == [[3, 4, 5]]
    out = torch.zeros(2, 3, dtype=torch.int32)
    staging.upload(table, out=out)
    assert out.tolist() == [[0, 1, 2], [99, 4, 5]]
    assert staging.fetch(torch.tensor([7, 8], dtype=torch.int32)).values() == [7, 8]


def test_token_log_lays_sequences_out_with_room():
    log = TokenLog("cpu", [[5, 6, 7], [], [9]], [2, 4, 0])
    assert log.begin == [0, 5, 9] and log.end == [5, 9, 10]
    assert log.tokens[:3].tolist() == [5, 6, 7] and int(log.tokens[9]) == 9
    # the sampler refuses a row whose log is full, before any kernel runs
    sampler = Sampler(EmulatedOps(), "cpu")
    config = SamplerConfig(temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.5)
    logits = torch.zeros(1, 16)
    with pytest.raises(ValueError, match="no room"):
        sampler.launch(logits, [config], [[9]], [0.0], log=(log, [2]))
    picked = sampler.launch(logits, [config], [[5, 6, 7]], [0.0], log=(log, [0]))
    assert int(log.tokens[3]) == int(picked[0])                 # the chosen token was appended behind the sequence's three
