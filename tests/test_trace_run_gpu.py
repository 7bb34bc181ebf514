"""bin/trace_run as a user runs it: the same requests replayed whole, with the last 32
tokens decoded one by one, and in batches of unequal lengths through reused slots, in
32-bit and in bfloat16; every logits file is compared with the plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from conftest import ROOT, TINY, WHOLE_ROTATION, make_folder
from helpers import assert_logits, token_ids
import plain_llama as P

pytestmark = pytest.mark.gpu


def replay(folder, dtype, out, steps, max_tokens):
    """Run bin/trace_run over `steps`; returns {step: array [wanted, vocab]}."""
    text = "".join(json.dumps(step) + "\n" for step in steps)
    done = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                           "--out", str(out), "--max-tokens", str(max_tokens)],
                          input=text, capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    lines = [line for line in done.stdout.splitlines() if line.startswith("done ")]
    assert lines == [f"done {step['step']}" for step in steps]
    vocab = json.load(open(os.path.join(folder, "config.json")))["vocab_size"]
    result = {}
    for step in steps:
        path = os.path.join(str(out), f"{step['step']}.f32")
        wanted = sum(len(e.get("want", [])) for e in step["entries"])
        assert os.path.exists(path) == (wanted > 0)
        if wanted:
            result[step["step"]] = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(wanted, vocab))
    return result


def trace_whole(requests):
    return [{"step": i, "entries": [{"id": name, "tokens": ids, "want": list(range(len(ids)))}], "end": [name]}
            for i, (name, ids) in enumerate(requests.items())]


def trace_tail(requests, tail=32):
    steps = []
    for name, ids in requests.items():
        head = max(1, len(ids) - tail)
        steps.append({"step": len(steps), "entries": [{"id": name, "tokens": ids[:head], "want": list(range(head))}], "end": []})
        for t in range(head, len(ids)):
            steps.append({"step": len(steps), "entries": [{"id": name, "tokens": [ids[t]], "want": [0]}],
                          "end": [name] if t == len(ids) - 1 else []})
        if head == len(ids):
            steps[-1]["end"] = [name]
    return steps


def trace_batches(batches, prompt_of):
    """Each batch starts together with unequal prompts, then one token per live request; a
    request ends after its last token; the next batch starts when the batch is over."""
    steps = []
    for batch in batches:
        at = {name: prompt_of(name, ids) for name, ids in batch.items()}
        entries = [{"id": n, "tokens": ids[:at[n]], "want": list(range(at[n]))} for n, ids in batch.items()]
        steps.append({"step": len(steps), "entries": entries, "end": [n for n, ids in batch.items() if at[n] == len(ids)]})
        while any(at[n] < len(ids) for n, ids in batch.items()):
            live = [n for n, ids in batch.items() if at[n] < len(ids)]
            entries = [{"id": n, "tokens": [batch[n][at[n]]], "want": [0]} for n in live]
            for n in live:
                at[n] += 1
            steps.append({"step": len(steps), "entries": entries, "end": [n for n in live if at[n] == len(batch[n])]})
    return steps


def collect(steps, outputs):
    """{request: logits [len, vocab]} from the files of a replay."""
    rows = {}
    for step in steps:
        if step["step"] not in outputs:
            continue
        at = 0
        for entry in step["entries"]:
            n = len(entry["want"])
            rows.setdefault(entry["id"], []).append(outputs[step["step"]][at:at + n])
            at += n
    return {name: torch.cat(parts) for name, parts in rows.items()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["llama", "qwen3"])
def test_replay_schedules(name, dtype, tmp_path):
    folder = make_folder(TINY[name], tmp_path / "model", seed=13, std=0.2)
    plain = P.PlainModel(folder)
    vocab = plain.config.vocab_size
    lengths = {"a": 40, "b": 7, "c": 100, "d": 65, "e": 1, "f": 90}
    requests = {n: token_ids(vocab, length, seed=length) for n, length in lengths.items()}
    want = {n: plain.logits(ids) for n, ids in requests.items()}

    whole = trace_whole(requests)
    got_whole = collect(whole, replay(folder, dtype, tmp_path / "whole", whole, 128))
    tail = trace_tail(requests)
    got_tail = collect(tail, replay(folder, dtype, tmp_path / "tail", tail, 128))
    names = list(requests)
    batches = [{n: requests[n] for n in names[:3]}, {n: requests[n] for n in names[3:]}]
    batched = trace_batches(batches, lambda n, ids: max(1, len(ids) - 5 - ord(n) % 3))
    # 64 + 64 + 128 tokens are held by the first batch at its fullest
    got_batched = collect(batched, replay(folder, dtype, tmp_path / "batched", batched, 256))
    for n in names:
        assert_logits(got_whole[n], want[n], dtype, f"{name} whole {n}")
        assert_logits(got_tail[n], want[n], dtype, f"{name} tail {n}")
        assert_logits(got_batched[n], want[n], dtype, f"{name} batched {n}")
        if dtype == "float32":
            assert torch.equal(got_whole[n], got_tail[n]) and torch.equal(got_whole[n], got_batched[n])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("head_dim", [64, 128])
def test_replay_in_portions(head_dim, dtype, tmp_path):
    """A request fed in portions of several tokens (the matrix-core attention at head sizes 64 and 128 continues
    a sequence in the middle of its cache): a portion that ends at a block's end, so that the next starts on a
    block's boundary; a portion of two tokens; one that ends at a block's end again; then token by token, while
    a second request of the same steps starts later and runs beside it."""
    raw = dict(TINY["qwen3" if head_dim == 128 else "llama"], hidden_size=128, num_attention_heads=2, num_key_value_heads=1,
               head_dim=head_dim, max_position_embeddings=512, **WHOLE_ROTATION)
    # (weights of std 0.1: at this width std 0.2 makes scores so large that their rounding to bfloat16 alone moves
    # logits by 5 % of the largest, in the kernels as in the stand-in that only rounds where they round)
    folder = make_folder(raw, tmp_path / "model", seed=head_dim, std=0.1)
    plain = P.PlainModel(folder)
    vocab = plain.config.vocab_size
    ids, other = token_ids(vocab, 230, seed=1), token_ids(vocab, 150, seed=2)
    cuts = [0, 64, 66, 192, 225, 226, 227, 228, 229, 230]
    steps = []
    for index, (begin, end) in enumerate(zip(cuts, cuts[1:])):
        entries = [{"id": "a", "tokens": ids[begin:end], "want": list(range(end - begin))}]
        if index >= 2:                   # the second request: one portion a step, of other sizes
            first, last = (index - 2) * 21, min(150, (index - 1) * 21)
            entries.append({"id": "b", "tokens": other[first:last], "want": list(range(last - first))})
        steps.append({"step": index, "entries": entries, "end": ["a", "b"] if end == 230 else []})
    assert (len(cuts) - 3) * 21 >= 147
    got = collect(steps, replay(folder, dtype, tmp_path / "portions", steps, 512))
    assert_logits(got["a"], plain.logits(ids), dtype, f"head {head_dim}: a request in portions")
    assert_logits(got["b"], plain.logits(other)[:got["b"].shape[0]], dtype, f"head {head_dim}: a request in portions beside it")
    if dtype == "float32":
        whole = trace_whole({"a": ids})
        assert torch.equal(collect(whole, replay(folder, dtype, tmp_path / "whole", whole, 512))["a"], got["a"])


def test_replay_without_wanted_logits_writes_no_file(tmp_path):
    folder = make_folder(TINY["llama"], tmp_path / "model", seed=1)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": [1, 2, 3], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": [4], "want": [0]}], "end": ["x"]}]
    out = replay(folder, "float32", tmp_path / "out", steps, 64)
    assert list(out) == [1]
    assert_logits(out[1], P.PlainModel(folder).logits([1, 2, 3, 4])[3:], "float32")


def test_command_line_generates_what_the_plain_loop_does(tmp_path):
    folder = make_folder(TINY["qwen3"], tmp_path / "model", seed=21, std=0.2)
    plain = P.PlainModel(folder)
    prompts = [[5, 9, 2], [100, 101, 102, 103, 104, 105, 106], []]
    command = [sys.executable, os.path.join(ROOT, "bin", "xrt"), "generate", "--model", folder, "--dtype", "float32",
               "--max-tokens", "7", "--temperature", "0", "--repetition-penalty", "1.0", "--stop-ids", "",
               "--prompt-ids", "5,9,2;100 101 102 103 104 105 106", "--prompt-ids", ""]
    done = subprocess.run(command, capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    lines = [[int(t) for t in line.split()] for line in done.stdout.strip().splitlines()]
    assert lines == [P.generate_greedy(plain, p, 7, stop_ids=[]) for p in prompts]
    assert "tokens in" in done.stderr and "decode" in done.stderr and "tok/s" in done.stderr
    # the repetition penalty of the reference's defaults reaches the kernel: it changes greedy output
    penalised = subprocess.run(command[:11] + ["--repetition-penalty", "5.0", "--stop-ids", "", "--prompt-ids", "5,9,2"],
                               capture_output=True, text=True, timeout=300)
    assert penalised.returncode == 0, penalised.stderr[-2000:]
    got = [int(t) for t in penalised.stdout.split()]
    assert got == P.generate_greedy(plain, prompts[0], 7, stop_ids=[], repetition_penalty=5.0)
    assert got != lines[0]
