"""The engine at the layer sizes of real models (Llama-3-8B, Qwen3-8B, Qwen3-32B, Llama-3.2-1B and Qwen3-0.6B
shapes, two layers of them) and at a context of 4096, against the plain implementation, in 32-bit and in bfloat16.

Weights come from the random-weights mode in memory (`Engine.random`); the plain model gets the
same tensors through `get_tensor`, which makes them again on the host. Schedules: a prompt alone
and whole; a slot filled to 4096 - 40 tokens in portions (one starts on a block's boundary, one
has two tokens, one ends at a block's end) and then 40 tokens one by one; an unequal batch of 72
requests that shrinks through every kernel's range of rows as requests end, then a second batch
through the same slots. These are the sizes at which the decode attention cuts its keys into
parts, the products of 17 to 64 rows split along k = 14336, and the big tiles run inside a model.
"""
import pytest
import torch

from helpers import assert_logits, errors, first_bad_position, plain_matrix, token_ids
import plain_llama as P

pytestmark = pytest.mark.gpu

SHAPES = {
    "llama3-8b": dict(architectures=["LlamaForCausalLM"], vocab_size=128256, hidden_size=4096, intermediate_size=14336,
                      num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                      rms_norm_eps=1e-5, rope_theta=500000.0, max_position_embeddings=4096,
                      tie_word_embeddings=False, hidden_act="silu"),
    "qwen3-8b": dict(architectures=["Qwen3ForCausalLM"], vocab_size=151936, hidden_size=4096, intermediate_size=12288,
                     num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                     rms_norm_eps=1e-6, rope_theta=1000000.0, max_position_embeddings=4096,
                     tie_word_embeddings=False, hidden_act="silu"),
    # a width that is no power of two, groups of eight query heads, products of k = 25600
    "qwen3-32b": dict(architectures=["Qwen3ForCausalLM"], vocab_size=151936, hidden_size=5120, intermediate_size=25600,
                      num_hidden_layers=2, num_attention_heads=64, num_key_value_heads=8, head_dim=128,
                      rms_norm_eps=1e-6, rope_theta=1000000.0, max_position_embeddings=4096,
                      tie_word_embeddings=False, hidden_act="silu"),
    # small shapes: heads of 64 with a width of 2048 (matrices with too few rows to be kept packed), a tied head
    "llama32-1b": dict(architectures=["LlamaForCausalLM"], vocab_size=128256, hidden_size=2048, intermediate_size=8192,
                       num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=8, head_dim=64,
                       rms_norm_eps=1e-5, rope_theta=500000.0, max_position_embeddings=4096,
                       tie_word_embeddings=True, hidden_act="silu"),
    # heads that are wider together than the model (16 x 128 against 1024), head norms, a tied head
    "qwen3-0.6b": dict(architectures=["Qwen3ForCausalLM"], vocab_size=151936, hidden_size=1024, intermediate_size=3072,
                       num_hidden_layers=2, num_attention_heads=16, num_key_value_heads=8, head_dim=128,
                       rms_norm_eps=1e-6, rope_theta=1000000.0, max_position_embeddings=4096,
                       tie_word_embeddings=True, hidden_act="silu"),
}
LAYERS_OF_THE_MODELS = {"llama3-8b": 32, "qwen3-8b": 36, "qwen3-32b": 64, "llama32-1b": 16, "qwen3-0.6b": 28}   # the tests run two layers of these sizes
CONTEXT, TAIL = 4096, 40
PORTIONS = [1024, 2, 2046, 984]             # 4056 tokens: a start on a block's boundary, two tokens, an end at a block's end
WHOLE = 300
SEED = {"llama3-8b": 3, "qwen3-8b": 4, "qwen3-32b": 5, "llama32-1b": 6, "qwen3-0.6b": 7}


def batch_plan(vocab):
    """72 requests of a first batch and 20 of a second: (tokens, prompt length) each. Prompts of 1 to 64
    tokens, 1 to 24 decoded tokens, so the batch passes 64, 16 and fewer rows as it drains."""
    generator = torch.Generator().manual_seed(21)
    plans = []
    for count in (72, 20):
        prompts = torch.randint(1, 65, (count,), generator=generator).tolist()
        decoded = torch.randint(1, 25, (count,), generator=generator).tolist()
        prompts[0], prompts[1], decoded[0], decoded[1] = 64, 1, 24, 24
        plans.append([(token_ids(vocab, p + d, seed=1000 + 100 * count + i), p)
                      for i, (p, d) in enumerate(zip(prompts, decoded))])
    return plans


def run_plan(engine, plan):
    """All requests of `plan` start together with their prompts and go on one token a step; a request
    whose tokens are used up frees its slot while the others go on. Logits of every request from its
    prompt's last position on."""
    slots = [engine.alloc_slot() for _ in plan]
    rows = [[] for _ in plan]
    logits = engine.step([(slot, ids[:p], [p - 1]) for slot, (ids, p) in zip(slots, plan)])
    for i in range(len(plan)):
        rows[i].append(logits[i:i + 1].cpu())
    position = [p for _, p in plan]
    live = list(range(len(plan)))
    while True:
        for i in [i for i in live if position[i] >= len(plan[i][0])]:
            engine.free_slot(slots[i])
            live.remove(i)
        if not live:
            break
        logits = engine.step([(slots[i], [plan[i][0][position[i]]], [0]) for i in live]).cpu()
        for row, i in enumerate(live):
            rows[i].append(logits[row:row + 1])
            position[i] += 1
    return [torch.cat(r) for r in rows]


@pytest.fixture(scope="module", params=list(SHAPES))
def case(request):
    """(shape name, configuration, {dtype: references}): the plain model's logits for every schedule, with
    the weights as the model of that dtype holds them (bfloat16: rounded once, then exact)."""
    from xeno_rt_amd.config import parse_config
    from xeno_rt_amd.weights import make_tensor
    from xeno_rt_amd.config import architecture

    name = request.param
    config = parse_config(SHAPES[name])
    specs = architecture(config.architecture).build(config).weight_specs()
    wide = {n: make_tensor(s, SEED[name], n, 0.02, torch.float32, gain_std=0.1) for n, s in specs.items()}
    vocab = config.vocab_size
    whole_ids = token_ids(vocab, WHOLE, seed=5)
    long_ids = token_ids(vocab, CONTEXT, seed=6)
    plans = batch_plan(vocab)
    references = {}
    for dtype in ("float32", "bfloat16"):
        weights = wide if dtype == "float32" else {n: t.to(torch.bfloat16).float() for n, t in wide.items()}
        plain = P.PlainModel.from_weights(SHAPES[name], weights)
        references[dtype] = dict(
            whole=plain.logits(whole_ids),
            long=plain.logits(long_ids, tail=TAIL + 1),
            batches=[[plain.logits(ids, tail=len(ids) - p + 1) for ids, p in plan] for plan in plans])
        del plain, weights
    return name, config, dict(whole_ids=whole_ids, long_ids=long_ids, plans=plans, references=references, wide=wide)


@pytest.fixture(scope="module")
def engines(case):
    from xeno_rt_amd.engine import Engine
    name, config, _ = case
    made = {}

    def get(dtype):
        if dtype not in made:
            made.clear()                    # one model of these sizes on the device at a time
            torch.cuda.empty_cache()
            made[dtype] = Engine.random(config, seed=SEED[name], dtype=dtype, std=0.02, gain_std=0.1,
                                        max_tokens=CONTEXT + 72 * 128, max_slots=72)
        return made[dtype]
    return get


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_weights_made_on_the_device_are_those_made_on_the_host(case, engines, dtype):
    name, config, data = case
    engine = engines(dtype)
    kind = torch.float32 if dtype == "float32" else torch.bfloat16
    mixer = engine.model.spec.layers[1].mixer
    p = "model.layers.1.self_attn."
    want = torch.cat([data["wide"][p + f"{n}_proj.weight"] for n in "qkv"]).to(kind)
    assert torch.equal(plain_matrix(mixer.w_qkv).cpu(), want)
    head = "model.embed_tokens.weight" if config.tie_word_embeddings else "lm_head.weight"
    assert torch.equal(plain_matrix(engine.model.spec.head.weight).cpu(), data["wide"][head].to(kind))
    if dtype == "bfloat16" and config.hidden_size >= 4096:          # matrices of these sizes are kept in tiles, for the products of few rows
        assert hasattr(mixer.w_qkv, "unpacked") and hasattr(engine.model.spec.layers[0].feed_forward.w_gate_up, "unpacked")
    gain = engine.model.spec.layers[0].feed_forward_norm.weight
    assert torch.equal(gain.cpu().float(), data["wide"]["model.layers.0.post_attention_layernorm.weight"].to(gain.dtype).float())
    assert torch.equal(engine.get_tensor("model.layers.0.mlp.down_proj.weight"),
                       data["wide"]["model.layers.0.mlp.down_proj.weight"].to(kind))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_prompt_alone_and_whole(case, engines, dtype):
    name, config, data = case
    engine = engines(dtype)
    slot = engine.alloc_slot()
    got = engine.step([(slot, data["whole_ids"], list(range(WHOLE)))])
    engine.free_slot(slot)
    want = data["references"][dtype]["whole"]
    worst, rms = assert_logits(got, want, dtype, f"{name} whole prompt, first bad row {first_bad_position(got, want, dtype)}")
    print(f"margins {name} {dtype} whole: max {worst:.2e} rms {rms:.2e}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_context_4096_filled_in_portions_then_token_by_token(case, engines, dtype):
    name, config, data = case
    engine = engines(dtype)
    ids = data["long_ids"]
    slot = engine.alloc_slot()
    at, rows = 0, []
    for index, count in enumerate(PORTIONS):
        last = index == len(PORTIONS) - 1
        logits = engine.step([(slot, ids[at:at + count], [count - 1] if last else [])])
        at += count
        if last:
            rows.append(logits)
    assert at == CONTEXT - TAIL
    for t in range(at, CONTEXT):
        rows.append(engine.step([(slot, [ids[t]], [0])]))
    assert engine.length(slot) == CONTEXT
    engine.free_slot(slot)
    got = torch.cat(rows)
    want = data["references"][dtype]["long"]
    worst, rms = assert_logits(got, want, dtype, f"{name} context 4096, first bad row {first_bad_position(got, want, dtype)}")
    print(f"margins {name} {dtype} context 4096: max {worst:.2e} rms {rms:.2e}")
    # the same rows from one step with all 4096 tokens: equal bit for bit in 32-bit, by tolerance in bfloat16
    slot = engine.alloc_slot()
    whole = engine.step([(slot, ids, list(range(CONTEXT - TAIL - 1, CONTEXT)))])
    engine.free_slot(slot)
    if dtype == "float32":
        assert torch.equal(whole, got), f"{name}: cutting the context into steps changed float32 bits"
    else:
        assert_logits(whole, want, dtype, f"{name} context 4096 in one step")
    engine.cache.check()
    assert engine.cache.held_blocks() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batch_of_72_that_drains_then_another_through_the_same_slots(case, engines, dtype):
    name, config, data = case
    engine = engines(dtype)
    worst_seen = rms_seen = 0.0
    for plan, wants in zip(data["plans"], data["references"][dtype]["batches"]):
        got = run_plan(engine, plan)
        for index, (logits, want, (ids, p)) in enumerate(zip(got, wants, plan)):
            worst, rms = assert_logits(logits, want, dtype,
                                       f"{name} batch of {len(plan)}, request {index} ({p} + {len(ids) - p} tokens), "
                                       f"first bad row {first_bad_position(logits, want, dtype)}")
            worst_seen, rms_seen = max(worst_seen, worst), max(rms_seen, rms)
        engine.cache.check()
        assert engine.cache.slots.n_held == 0 and engine.cache.held_blocks() == 0
        if dtype == "float32":
            # alone and whole: the same bits as in the batch
            for index in (0, 1, len(plan) // 2, len(plan) - 1):
                ids, p = plan[index]
                slot = engine.alloc_slot()
                alone = engine.step([(slot, ids, list(range(p - 1, len(ids))))]).cpu()
                engine.free_slot(slot)
                assert torch.equal(alone, got[index]), f"{name} request {index}: batching changed float32 bits"
    print(f"margins {name} {dtype} batches: max {worst_seen:.2e} rms {rms_seen:.2e}")
