"""The toy architecture of test_parts_gpu.py (a mixer with state of its own, another position encoding, a
feed-forward with routing, a layer that runs twice, a layer that reads another's cache) registered, built,
stepped and generated from on the CPU, with the test stand-in for the kernels: nothing of it needs the GPU
or a change to the framework's files."""
import torch

from helpers import assert_greedy_tokens, assert_logits, run_batched, run_tail_decoded, run_whole, token_ids
from ops_emulation import EmulatedOps
from test_parts_gpu import attention_with_scores_biased_by_distance, define_toy, plain_toy


def test_toy_architecture_on_the_cpu_stand_in(tmp_path):
    from xeno_rt_amd.config import load_config
    from xeno_rt_amd.engine import Engine, GenerateRequest, generate
    from xeno_rt_amd.weights import SafetensorsFile, write_random_model

    config = define_toy()
    folder = str(tmp_path / "toy")
    write_random_model(config, folder, seed=3, std=0.25)
    assert load_config(folder) == config
    engine = Engine.load(folder, dtype="float32", device="cpu", ops=EmulatedOps(), max_tokens=256, max_slots=3)
    assert engine.graphs is None                    # the toy mixer looks at the batch on the host: every step runs directly
    with SafetensorsFile(folder + "/model.safetensors") as file:
        w = {n: file.read(n).double() for n in file.names()}
    requests = [token_ids(150, n, seed=n) for n in (40, 9, 70)]
    want = [plain_toy(w, config, ids) for ids in requests]
    for ids, logits in zip(requests, want):
        assert_logits(run_whole(engine, ids), logits, "float32", "toy whole")
    assert_logits(run_tail_decoded(engine, requests[0]), want[0], "float32", "toy decoded tail")
    for got, logits in zip(run_batched(engine, requests, [20, 9, 30]), want):
        assert_logits(got, logits, "float32", "toy batch")
    out = generate(engine, [GenerateRequest(requests[1][:5], max_tokens=4, temperature=0.0, repetition_penalty=1.0),
                            GenerateRequest(requests[2][:3], max_tokens=6, temperature=0.0, repetition_penalty=1.3)])
    assert [len(o.tokens) for o in out] == [4, 6]
    logits_of = lambda ids: plain_toy(w, config, ids)
    assert_greedy_tokens(logits_of, requests[1][:5], out[0].tokens, "float32", 1.0, "toy generation")
    assert_greedy_tokens(logits_of, requests[2][:3], out[1].tokens, "float32", 1.3, "toy generation with a penalty")
    engine.cache.check()
    assert engine.cache.slots.n_held == 0


def test_a_position_encoding_on_the_scores_on_the_cpu_stand_in():
    from xeno_rt_amd.parts import Runtime
    got, want, unbiased = attention_with_scores_biased_by_distance(Runtime(EmulatedOps(), torch.float32, "cpu"), "float32", "cpu")
    error = float((got.double() - want).abs().max()) / float(want.abs().max())
    assert error < 2e-5
    assert float((unbiased - want).abs().max()) / float(want.abs().max()) > 1e-3
