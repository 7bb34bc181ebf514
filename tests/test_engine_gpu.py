"""The engine on the GPU against the plain implementation: whole requests, decoded tails,
unequal batches with slot reuse, long decoding, first tokens, greedy generation; in 32-bit
and in bfloat16, for two tiny configurations that differ in every size and option."""
import pytest
import torch

from conftest import TINY, WHOLE_ROTATION, make_folder
from helpers import (TOLERANCE, assert_logits, errors, first_bad_position, run_batched, run_tail_decoded, run_whole,
                     token_ids)
import plain_llama as P

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
LENGTHS = {"llama": [5, 11, 17, 64, 65, 128], "qwen3": [1, 7, 23, 30, 129, 200]}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """name -> (folder, plain model, {length: (ids, plain logits)})"""
    out = {}
    for name in ("llama", "qwen3"):
        folder = make_folder(TINY[name], tmp_path_factory.mktemp(name), seed=31 if name == "llama" else 47, std=0.2)
        plain = P.PlainModel(folder)
        cases = {}
        for index, length in enumerate(LENGTHS[name]):
            ids = token_ids(plain.config.vocab_size, length, seed=100 + index)
            cases[length] = (ids, plain.logits(ids))
        out[name] = (folder, plain, cases)
    return out


@pytest.fixture(scope="module")
def engines(models):
    from xeno_rt_amd.engine import Engine
    cache = {}

    def get(name, dtype):
        if (name, dtype) not in cache:
            # eight blocks and three slots: batches must reuse both
            cache[(name, dtype)] = Engine.load(models[name][0], dtype=dtype, max_tokens=64 * 8, max_slots=3)
        return cache[(name, dtype)]
    return get


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["llama", "qwen3"])
def test_each_request_alone_and_whole(name, dtype, models, engines):
    engine = engines(name, dtype)
    for length, (ids, want) in models[name][2].items():
        got = run_whole(engine, ids)
        assert_logits(got, want, dtype, f"{name} whole length {length}, first bad row {first_bad_position(got, want, dtype)}")
    engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["llama", "qwen3"])
def test_last_32_tokens_one_by_one(name, dtype, models, engines):
    engine = engines(name, dtype)
    for length, (ids, want) in models[name][2].items():
        got = run_tail_decoded(engine, ids)
        assert_logits(got, want, dtype, f"{name} decoded tail length {length}, first bad row {first_bad_position(got, want, dtype)}")
        if dtype == "float32":
            # the 32-bit kernels sum in an order that does not depend on the step's shape
            assert torch.equal(got, run_whole(engine, ids)), f"{name} length {length}: cutting changed float32 bits"
    engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["llama", "qwen3"])
def test_unequal_batches_one_after_another(name, dtype, models, engines):
    engine = engines(name, dtype)
    cases = models[name][2]
    lengths = LENGTHS[name]
    # three batches through three slots; prompts are shorter than the requests, so the tail of
    # every request is decoded, and shorter requests end while longer ones go on
    batches = [lengths[0:3], lengths[3:5] + [lengths[1]], [lengths[5], lengths[0], lengths[2]]]
    for batch in batches:
        requests = [cases[n][0] for n in batch]
        prompts = [max(1, n - 1 - 3 * i) for i, n in enumerate(batch)]
        got = run_batched(engine, requests, prompts)
        for n, logits in zip(batch, got):
            assert_logits(logits, cases[n][1], dtype,
                          f"{name} batch {batch} request of {n}, first bad row {first_bad_position(logits, cases[n][1], dtype)}")
            if dtype == "float32":
                assert torch.equal(logits, run_whole(engine, cases[n][0])), f"{name} {n}: batching changed float32 bits"
        engine.cache.check()
        assert engine.cache.slots.n_held == 0 and engine.cache.held_blocks() == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["llama", "qwen3"])
def test_long_decoding_from_the_first_token(name, dtype, models, engines):
    engine = engines(name, dtype)
    folder, plain, _ = models[name]
    length = plain.config.max_position            # up to the last position of the context
    ids = token_ids(plain.config.vocab_size, length, seed=9)
    want = plain.logits(ids)
    got = run_tail_decoded(engine, ids, tail=length - 1)      # one token, then all others one by one
    assert_logits(got[:4], want[:4], dtype, f"{name} first tokens")
    assert_logits(got, want, dtype, f"{name} long decoding, first bad row {first_bad_position(got, want, dtype)}")
    assert engine.cache.held_blocks() == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["llama", "qwen3"])
def test_greedy_generation_through_the_entry_point(name, dtype, models, engines):
    from xeno_rt_amd.engine import GenerateRequest, generate
    engine = engines(name, dtype)
    folder, plain, cases = models[name]
    prompts = [cases[n][0] for n in LENGTHS[name][:4]] + [[]]
    limits = [9, 14, 5, 12, 4]
    requests = [GenerateRequest(p, max_tokens=n, temperature=0.0, repetition_penalty=1.0, stop_ids=[])
                for p, n in zip(prompts, limits)]
    results = generate(engine, requests, batch_size=3)
    bos = [plain.config.bos_id]

    def check(prompt, tokens):
        if dtype == "float32":
            assert tokens == P.generate_greedy(plain, prompt, len(tokens), stop_ids=[])
            return
        # bfloat16 may pick another of two near-equal logits (and which one can depend on the
        # batch, whose size selects the kernel and with it the order of the sums): every chosen
        # token must be the plain model's best within the tolerance, given the tokens before it
        history = list(prompt or bos)
        for token in tokens:
            row = plain.logits(history)[-1]
            assert float(row.max() - row[token]) <= 2 * TOLERANCE[dtype]["max"] * float(row.abs().max())
            history.append(token)

    for prompt, limit, result in zip(prompts, limits, results):
        assert len(result.tokens) == limit and result.finish_reason == "length"
        check(prompt, result.tokens)
    # stop tokens: the request ends before the token, the others go on
    free = results[1].tokens
    again = generate(engine, [GenerateRequest(prompts[1], max_tokens=14, temperature=0.0, repetition_penalty=1.0,
                                              stop_ids=[free[5]]),
                              GenerateRequest(prompts[0], max_tokens=9, temperature=0.0, repetition_penalty=1.0,
                                              stop_ids=[])])
    assert free[5] not in again[0].tokens and len(again[1].tokens) == 9     # a stop token is never returned
    check(prompts[1], again[0].tokens)
    check(prompts[0], again[1].tokens)
    if dtype == "float32":
        assert again[0].finish_reason == "stop"
        assert again[0].tokens == free[:free.index(free[5])] and again[1].tokens == results[0].tokens
    engine.cache.check()
    assert engine.cache.slots.n_held == 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_far_keys_among_hundreds(dtype, tmp_path):
    """Several hundred tokens of context with weights that make attention sharp: the keys that
    matter lie far back, in other cache blocks than the query.

    Weights this sharp (std 0.3) turn the rounding of q and k to bfloat16 into errors of up to 6 % of
    the largest logit, whatever computes them: the stand-in for the kernels, which rounds where they
    round and otherwise computes in float32 on the host, is as far from the plain model as the kernels
    are. The bfloat16 engine is therefore compared with that stand-in (a key that is missed or read from
    the wrong block moves logits by far more than the orders of summation do), the 32-bit engine with
    the plain model."""
    from ops_emulation import EmulatedOps
    from xeno_rt_amd.engine import Engine
    raw = dict(TINY["llama"], max_position_embeddings=1024, num_hidden_layers=1, rope_theta=50000.0)
    folder = make_folder(raw, tmp_path / "far", seed=5, std=0.3)
    plain = P.PlainModel(folder)
    ids = token_ids(plain.config.vocab_size, 700, seed=3)
    want = plain.logits(ids)
    if dtype == "bfloat16":
        rounded = run_whole(Engine.load(folder, dtype=dtype, max_tokens=1024, device="cpu", ops=EmulatedOps()), ids)
        worst, rms = errors(rounded, want)
        assert worst < 0.1 and rms < 0.01, "the stand-in itself is off"
        want = rounded
    engine = Engine.load(folder, dtype=dtype, max_tokens=1024)
    whole = run_whole(engine, ids)
    assert_logits(whole, want, dtype, "700 tokens whole")
    got = run_tail_decoded(engine, ids)
    assert_logits(got, want, dtype, f"700 tokens, tail decoded, first bad row {first_bad_position(got, want, dtype)}")
    if dtype == "bfloat16":
        # and against the plain model itself, so that the engine has a bound that does not hang on the stand-in:
        # what is asked of the stand-in above, and the plain model's choice of token in nearly every row
        plain_logits = plain.logits(ids)
        for what, rows in (("whole", whole), ("tail decoded", got)):
            worst, rms = errors(rows, plain_logits)
            assert worst < 0.1 and rms < 0.01, f"700 tokens {what} against the plain model: max {worst:.3e}, rms {rms:.3e}"
            same = (rows.argmax(-1).cpu() == plain_logits.argmax(-1)).float().mean()
            assert float(same) > 0.9, f"700 tokens {what}: the plain model's token in only {float(same):.2f} of the rows"


@pytest.mark.parametrize("dtype", DTYPES)
def test_replayed_decode_steps_equal_direct_ones(dtype, models):
    """Decode steps run as recorded graphs; every replay must give the bits of the same step run
    directly, with other work (a prompt of another sequence, host synchronisation, a batch that
    shrinks and so changes the graph) between the replays."""
    from xeno_rt_amd.engine import Engine
    folder, plain, _ = models["qwen3"]
    vocab = plain.config.vocab_size
    recorded = Engine.load(folder, dtype=dtype, max_tokens=64 * 12, max_slots=4)
    direct = Engine.load(folder, dtype=dtype, max_tokens=64 * 12, max_slots=4, graphs=False)
    assert recorded.graphs is not None and direct.graphs is None
    prompts = [token_ids(vocab, n, seed=n) for n in (3, 70, 129)]
    outputs = []
    for engine in (recorded, direct):
        rows = []
        slots = [engine.alloc_slot() for _ in prompts]
        rows.append(engine.step([(s, p, [len(p) - 1]) for s, p in zip(slots, prompts)]))
        live = list(range(3))
        for step in range(70):
            tokens = token_ids(vocab, len(live), seed=1000 + step)
            rows.append(engine.step([(slots[i], [tokens[j]], [0]) for j, i in enumerate(live)]))
            if step % 9 == 4:                       # other work between replays: a new sequence comes and goes
                extra = engine.alloc_slot()
                rows.append(engine.step([(extra, token_ids(vocab, 40, seed=step), [39])]))
                engine.free_slot(extra)
                torch.cuda.synchronize()
            if step == 30:                          # the shortest request ends: the batch, and the graph, change
                engine.free_slot(slots[live.pop(0)])
        for i in live:
            engine.free_slot(slots[i])
        outputs.append([r.clone() for r in rows])
    assert len(recorded.graphs.graphs) >= 2
    for index, (a, b) in enumerate(zip(*outputs)):
        assert torch.equal(a, b), f"step {index}: a replayed graph differs from the direct step"


@pytest.mark.parametrize("dtype", DTYPES)
def test_recorded_steps_share_memory_and_make_room_for_each_other(dtype, models, monkeypatch):
    """All recorded steps draw on one memory pool and at most MAX_GRAPHS are kept: steps of three
    shapes taken in turn (each replay between replays of the others, each shape recorded again after
    it had to make room) give the bits of direct steps."""
    from xeno_rt_amd.engine import Engine, graphs
    monkeypatch.setattr(graphs, "MAX_GRAPHS", 2)
    folder, plain, _ = models["llama"]
    vocab = plain.config.vocab_size
    recorded = Engine.load(folder, dtype=dtype, max_tokens=64 * 16, max_slots=8)
    direct = Engine.load(folder, dtype=dtype, max_tokens=64 * 16, max_slots=8, graphs=False)
    outputs = []
    for engine in (recorded, direct):
        rows = []
        slots = [engine.alloc_slot() for _ in range(7)]
        engine.step([(slot, token_ids(vocab, 5 + 9 * i, seed=i), []) for i, slot in enumerate(slots)])
        for step in range(24):
            live = slots[:(1, 3, 7)[step % 3]]                   # batch buckets 1, 4 and 8 in turn
            tokens = token_ids(vocab, len(live), seed=300 + step)
            rows.append(engine.step([(slot, [token], [0]) for slot, token in zip(live, tokens)]))
        for slot in slots:
            engine.free_slot(slot)
        outputs.append(rows)
    assert len(recorded.graphs.graphs) == 2
    for index, (a, b) in enumerate(zip(*outputs)):
        assert torch.equal(a, b), f"step {index}: a replayed graph differs from the direct step"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["llama", "qwen3"])
def test_a_step_may_mix_sequences_that_start_with_sequences_that_go_on(name, dtype, models, engines):
    """One step with a whole prompt of a new sequence, one token of a sequence under way, and several
    tokens of another one under way (its start not on a block's boundary)."""
    engine = engines(name, dtype)
    _, plain, cases = models[name]
    lengths = LENGTHS[name]
    a, b, c = (cases[n] for n in (lengths[3], lengths[4], lengths[5]))     # (ids, plain logits)
    slots = [engine.alloc_slot() for _ in range(3)]
    cut_b, cut_c = len(b[0]) - 1, len(c[0]) - 37
    first = engine.step([(slots[1], b[0][:cut_b], list(range(cut_b))), (slots[2], c[0][:cut_c], list(range(cut_c)))])
    mixed = engine.step([(slots[0], a[0], list(range(len(a[0])))),
                         (slots[1], b[0][cut_b:], [0]),
                         (slots[2], c[0][cut_c:], list(range(37)))])
    for slot in slots:
        engine.free_slot(slot)
    got_a = mixed[:len(a[0])]
    got_b = torch.cat([first[:cut_b], mixed[len(a[0]):len(a[0]) + 1]])
    got_c = torch.cat([first[cut_b:], mixed[len(a[0]) + 1:]])
    for what, got, (ids, want) in (("starting", got_a, a), ("one more token", got_b, b), ("37 more tokens", got_c, c)):
        assert_logits(got, want, dtype, f"{name} mixed step, the sequence {what}, first bad row {first_bad_position(got, want, dtype)}")
        if dtype == "float32":
            assert torch.equal(got, run_whole(engine, ids)), f"{name}: a mixed step changed float32 bits ({what})"
    engine.cache.check()


@pytest.mark.parametrize("arch,sizes", [
    ("llama", dict(num_attention_heads=4, num_key_value_heads=1, head_dim=64, max_position_embeddings=1200)),
    # half of a head rotated, positions halved: the projection's epilogue does not rotate such heads, a kernel after it does
    ("llama", dict(num_attention_heads=4, num_key_value_heads=2, head_dim=128, hidden_size=64, max_position_embeddings=1200,
                   partial_rotary_factor=0.5, rope_scaling={"rope_type": "linear", "factor": 2.0})),
    # with head norms and heads rotated whole, the attention of a bfloat16 decode step also norms and rotates q and the new key
    # and writes the cache (angles from a table, here of positions divided by 4, and of plain positions)
    ("qwen3", dict(num_attention_heads=6, num_key_value_heads=2, head_dim=128, max_position_embeddings=1200, **WHOLE_ROTATION)),
    ("qwen3", dict(num_attention_heads=6, num_key_value_heads=3, head_dim=64, max_position_embeddings=1200, rope_scaling=None, **WHOLE_ROTATION)),
    # head norms and half of a head rotated: the preparation kernel stays between projection and attention
    ("qwen3", dict(num_attention_heads=6, num_key_value_heads=2, head_dim=128, max_position_embeddings=1200)),
])
@pytest.mark.parametrize("dtype", DTYPES)
def test_decoding_across_a_thousand_tokens(dtype, arch, sizes, tmp_path):
    """Two sequences decode from just under 1024 tokens to beyond it, one of them from a block edge:
    the recorded decode steps change their context size on the way (head sizes 64 and 128: in bfloat16 the
    matrix-core decode kernel with its split over key chunks and its merge). Every step must equal
    the same step run directly, and the last logits must be the plain model's."""
    from xeno_rt_amd.engine import Engine
    raw = dict(TINY[arch], num_hidden_layers=2, rope_theta=50000.0, **sizes)
    folder = make_folder(raw, tmp_path / "long", seed=9, std=0.25)
    plain = P.PlainModel(folder)
    vocab = plain.config.vocab_size
    starts, steps = (1000, 960), 70
    sequences = [token_ids(vocab, n + steps, seed=n) for n in starts]
    rows = []
    for graphs in (True, False):
        engine = Engine.load(folder, dtype=dtype, max_tokens=64 * 40, max_slots=2, graphs=graphs)
        slots = [engine.alloc_slot() for _ in starts]
        engine.step([(s, ids[:n], []) for s, ids, n in zip(slots, sequences, starts)])
        out = [engine.step([(s, [ids[n + t]], [0]) for s, ids, n in zip(slots, sequences, starts)]).clone()
               for t in range(steps)]
        rows.append(out)
        if graphs:
            assert engine.graphs is not None and len(engine.graphs.graphs) >= 2     # two context sizes
    for t, (a, b) in enumerate(zip(*rows)):
        assert torch.equal(a, b), f"decode step {t}: the recorded step differs from the direct one"
    for i, (ids, n) in enumerate(zip(sequences, starts)):
        want = plain.logits(ids)[-1:]
        assert_logits(rows[0][-1][i:i + 1], want, dtype, f"sequence {i}, last decoded token")


@pytest.mark.parametrize("arch,head_dim", [("qwen3", 64), ("llama", 64), ("llama", 128)])
@pytest.mark.parametrize("dtype", DTYPES)
def test_a_batch_of_forty_sequences(dtype, arch, head_dim, tmp_path):
    """Forty sequences of unequal lengths start together and end one after the other: the step's
    token count runs through 300-odd (prompts), 40 and down to 1, and with a width of 128 the
    bfloat16 products take every kernel there is on the way: the tiled one and the one split along
    k for the prompts, the split one for 17 to 40 rows, the streaming one below (which, for up to 16 rows,
    also does the norms' work and, without head norms (llama), the rotation and the cache write)."""
    from xeno_rt_amd.engine import Engine
    raw = dict(TINY[arch], hidden_size=128, intermediate_size=320, num_attention_heads=4, num_key_value_heads=2,
               head_dim=head_dim, num_hidden_layers=2, max_position_embeddings=128, **WHOLE_ROTATION)
    folder = make_folder(raw, tmp_path / "wide", seed=13, std=0.15)
    plain = P.PlainModel(folder)
    vocab = plain.config.vocab_size
    lengths = [6 + (7 * i) % 45 for i in range(40)]
    prompts = [1 + (3 * i) % 5 + (i % 7) * 2 for i in range(40)]
    requests = [token_ids(vocab, n, seed=200 + i) for i, n in enumerate(lengths)]
    engine = Engine.load(folder, dtype=dtype, max_tokens=64 * 40, max_slots=40)
    got = run_batched(engine, requests, [min(p, n) for p, n in zip(prompts, lengths)])
    for i, (ids, rows) in enumerate(zip(requests, got)):
        assert_logits(rows, plain.logits(ids), dtype, f"request {i} of 40")
    engine.cache.check()
    assert engine.cache.slots.n_held == 0


@pytest.mark.parametrize("graphs", [True, False])
@pytest.mark.parametrize("dtype", DTYPES)
def test_generation_a_step_ahead_equals_generation_through_the_host(dtype, graphs, models, engines):
    """The loop starts a step from the sampled tokens on the device before it has seen them. The same
    requests, sampled with a temperature, through a loop written here that brings every token to the
    host first, with the same uniform numbers: the same tokens, also where a request draws a stop token
    (and has been stepped once for nothing) while the others go on."""
    from xeno_rt_amd.engine import GenerateRequest, generate
    from xeno_rt_amd.engine import Engine
    from xeno_rt_amd.sampling import Sampler, uniform
    # with recorded decode steps, and with every step run directly (as models do whose parts cannot be recorded)
    engine = engines("llama", dtype) if graphs else Engine.load(models["llama"][0], dtype=dtype, max_tokens=64 * 8,
                                                                max_slots=3, graphs=False)
    vocab = engine.config.vocab_size
    prompts = [token_ids(vocab, n, seed=300 + n) for n in (9, 3, 14)]
    # the second request has a repetition penalty: the loop keeps its tokens on the device, the loop below hands
    # them to the sampler at every step
    options = [dict(temperature=0.9, top_k=12, top_p=0.9, repetition_penalty=penalty) for penalty in (1.0, 1.3, 1.0)]

    def through_the_host(stops):
        sampler = Sampler(engine.ops, engine.device)
        configs = [GenerateRequest([], **o).sampler_config() for o in options]
        slots = [engine.alloc_slot() for _ in prompts]
        produced = [[] for _ in prompts]
        live = list(range(len(prompts)))
        logits = engine.step([(slots[i], prompts[i], [len(prompts[i]) - 1]) for i in live])
        while live:
            tokens = sampler.sample(logits, [configs[i] for i in live], [prompts[i] + produced[i] for i in live],
                                    [uniform(70 + i, 0, len(produced[i])) for i in live])
            still = []
            for i, token in zip(live, tokens):
                if token in stops:
                    continue
                produced[i].append(token)
                if len(produced[i]) < 24:
                    still.append(i)
            live = still
            if live:
                logits = engine.step([(slots[i], [produced[i][-1]], [0]) for i in live])
        for slot in slots:
            engine.free_slot(slot)
        return produced

    free = through_the_host(())
    # a stop token that the second request draws half-way, and that may end others too
    stop = free[1][10]
    want = through_the_host((stop,))
    assert len(want[1]) <= 10 and max(len(tokens) for tokens in want) > len(want[1]) + 1
    requests = [GenerateRequest(prompt, max_tokens=24, seed=70 + i, stop_ids=[stop], **options[i])
                for i, prompt in enumerate(prompts)]
    got = generate(engine, requests)
    assert [result.tokens for result in got] == want
    assert [result.finish_reason for result in got] == ["length" if len(t) == 24 else "stop" for t in want]
    engine.cache.check()
    assert engine.cache.slots.n_held == 0 and engine.cache.held_blocks() == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("arch,sizes", [
    ("llama", dict(hidden_size=400, num_attention_heads=4, num_key_value_heads=2, intermediate_size=232)),     # heads of 100, from hidden / heads
    ("qwen3", dict(hidden_size=96, num_attention_heads=4, num_key_value_heads=2, head_dim=72)),               # heads of 72, with head norms
    ("llama", dict(hidden_size=40, num_attention_heads=4, num_key_value_heads=4, intermediate_size=56)),      # heads of 10
])
def test_head_sizes_that_are_no_multiple_of_16(dtype, arch, sizes, tmp_path):
    """The reference takes any head size (llama.rs:125-128; the attention loops of :504-574 know no alignment):
    heads of 100, 72 and 10 dims, whole, with the tail decoded, and in a batch of unequal lengths."""
    from xeno_rt_amd.engine import Engine
    raw = dict(TINY[arch], max_position_embeddings=256, **sizes)
    folder = make_folder(raw, tmp_path / "heads", seed=19, std=0.08 if raw["hidden_size"] > 200 else 0.2)
    plain = P.PlainModel(folder)
    vocab = plain.config.vocab_size
    engine = Engine.load(folder, dtype=dtype, max_tokens=64 * 12, max_slots=3)
    requests = [token_ids(vocab, n, seed=500 + n) for n in (150, 70, 9)]
    wants = [plain.logits(ids) for ids in requests]
    for ids, want in zip(requests, wants):
        whole = run_whole(engine, ids)
        assert_logits(whole, want, dtype, f"{arch} {sizes} whole length {len(ids)}, first bad row {first_bad_position(whole, want, dtype)}")
        got = run_tail_decoded(engine, ids)
        assert_logits(got, want, dtype, f"{arch} {sizes} decoded tail length {len(ids)}, first bad row {first_bad_position(got, want, dtype)}")
        if dtype == "float32":
            assert torch.equal(got, whole), f"{arch} {sizes}: cutting changed float32 bits"
    got = run_batched(engine, requests, [100, 66, 1])
    for ids, logits, want in zip(requests, got, wants):
        assert_logits(logits, want, dtype, f"{arch} {sizes} batched, request of {len(ids)}")
    engine.cache.check()
    assert engine.cache.slots.n_held == 0 and engine.cache.held_blocks() == 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_step_of_a_size_seen_before_allocates_nothing_but_its_logits(dtype, models):
    """Steps that are launched kernel by kernel (prompts, and every step of a model whose steps cannot be recorded) cut
    their tensors, and the kernels' workspaces, from one stretch of memory that is as long as the largest step so far
    needed (the reference grows its scratch on demand and keeps it, llama.rs:240-268). What the caller gets (the
    logits) is memory of its own, and stays valid while later steps run."""
    from xeno_rt_amd.engine import Engine
    folder, plain, cases = models["qwen3"]
    engine = Engine.load(folder, dtype=dtype, max_tokens=64 * 8, max_slots=3, graphs=False)
    ids, want = cases[129]
    allocations = lambda: torch.cuda.memory_stats()["allocation.all.allocated"]
    kept = []
    for round_ in range(4):
        slot, other = engine.alloc_slot(), engine.alloc_slot()
        before = allocations()
        rows = [engine.step([(slot, ids[:100], list(range(100))), (other, ids[:7], [6])])]
        after_prompt = allocations()
        for t in range(100, 129):
            rows.append(engine.step([(slot, [ids[t]], [0]), (other, [ids[t - 93]], [])]))
        after_decoding = allocations()
        engine.free_slot(slot); engine.free_slot(other)
        if round_ >= 2:         # the first round finds out what a step needs, the second takes it once
            assert after_prompt - before == 1 and after_decoding - after_prompt == 29, \
                (after_prompt - before, after_decoding - after_prompt)
        kept.append(rows)
    for rows in kept:           # logits of earlier steps are still what they were
        got = torch.cat([rows[0][:100]] + rows[1:])
        assert_logits(got, want, dtype, "steps from the arena")
    assert torch.equal(torch.cat(kept[0]), torch.cat(kept[3]))
