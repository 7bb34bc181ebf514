"""Decode and prefill throughput of the dense decoder at the layer sizes of real models, random weights.

    python bench.py --gpus 1 --steps K --warmup W [--shape llama3-8b|qwen3-8b|qwen3-32b] [--dtype float32 --layers N]

A step is one decode step of the whole batch (8 sequences for the 8B shapes, 32 for the 32B shape,
unless --batch says otherwise): the engine's step function on one token per sequence, then greedy
sampling on the device. Every sequence's cache is first filled by real prefill steps so that the timed
steps end at the context length (4096). Beside the headline the record holds
  * one prefill of 2048 tokens (and, for the Qwen3-8B shape, one step with a batch of eight prompts of
    unequal lengths drawn from [64, 2048]), priced against the dense MFMA peak of the dtype;
  * the decode step priced against HBM: the bytes it has to read (every weight it uses once, and the
    cache of the live sequences) over its time, against the published 8 TB/s and against what a kernel
    that only reads reaches on this GPU (`measured_peak`); likewise the prefill against what the matrix
    cores reach on tiles that never leave the registers;
  * `points`: decoding at the other batch sizes of the shape and at a cache length of 128 (where only the
    weights count), each with tokens a second, ms a step and its fraction of the HBM bound;
  * `check`: the logits of one more decode step, run as the recorded graph and again directly (kernels
    launched one by one, no padding of batch or context), compared outside the timed region.
One JSON line goes to standard output; with more than one GPU asked for it says so and exits with 2.
"""
import argparse
import json
import sys
import time

import torch

PEAK_HBM_GBS = 8000.0           # MI355X HBM3E, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}   # dense MFMA, published

COMMON = dict(num_attention_heads=32, num_key_value_heads=8, head_dim=128, max_position_embeddings=8192,
              tie_word_embeddings=False, hidden_act="silu", torch_dtype="bfloat16")
SHAPES = {
    "llama3-8b": dict(COMMON, architectures=["LlamaForCausalLM"], vocab_size=128256, hidden_size=4096,
                      intermediate_size=14336, num_hidden_layers=32, rms_norm_eps=1e-5, rope_theta=500000.0),
    "qwen3-8b": dict(COMMON, architectures=["Qwen3ForCausalLM"], vocab_size=151936, hidden_size=4096,
                     intermediate_size=12288, num_hidden_layers=36, rms_norm_eps=1e-6, rope_theta=1000000.0),
    "qwen3-32b": dict(COMMON, architectures=["Qwen3ForCausalLM"], vocab_size=151936, hidden_size=5120,
                      intermediate_size=25600, num_hidden_layers=64, num_attention_heads=64, rms_norm_eps=1e-6,
                      rope_theta=1000000.0),
    # two small shapes: heads of 64, a tied output head, widths at which every kernel's fixed cost weighs most
    "llama32-1b": dict(COMMON, architectures=["LlamaForCausalLM"], vocab_size=128256, hidden_size=2048, head_dim=64,
                       intermediate_size=8192, num_hidden_layers=16, rms_norm_eps=1e-5, rope_theta=500000.0,
                       tie_word_embeddings=True),
    "qwen3-0.6b": dict(COMMON, architectures=["Qwen3ForCausalLM"], vocab_size=151936, hidden_size=1024,
                       num_attention_heads=16, intermediate_size=3072, num_hidden_layers=28, rms_norm_eps=1e-6,
                       rope_theta=1000000.0, tie_word_embeddings=True),
}
MODEL_NAMES = {"llama3-8b": "Llama-3-8B shape", "qwen3-8b": "Qwen3-8B shape", "qwen3-32b": "Qwen3-32B shape",
               "llama32-1b": "Llama-3.2-1B shape", "qwen3-0.6b": "Qwen3-0.6B shape"}
HEADLINE_BATCH = {"llama3-8b": 8, "qwen3-8b": 8, "qwen3-32b": 32, "llama32-1b": 8, "qwen3-0.6b": 8}
OTHER_BATCHES = {"llama3-8b": (1, 64), "qwen3-8b": (1, 64), "qwen3-32b": (1,), "llama32-1b": (1, 64), "qwen3-0.6b": (1, 64)}
CONTEXT = 4096
SHORT_CONTEXT = 128
PREFILL_TOKENS = 2048
LONG_PREFILL = 8192                # a second prefill point, where attention weighs more
UNEQUAL_PROMPTS = (8, 64, 2048)     # the Qwen3-8B shape's batch of prompts: count, shortest, longest


def weight_bytes(config, element):
    """Bytes of every weight that one decode step reads once (embedding rows are negligible)."""
    c = config
    per_layer = (c.q_width + 2 * c.kv_width) * c.hidden_size + c.hidden_size * c.q_width \
        + 3 * c.intermediate_size * c.hidden_size + 2 * c.hidden_size + (2 * c.head_dim if c.qk_norm else 0)
    return (c.num_hidden_layers * per_layer + c.hidden_size + c.vocab_size * c.hidden_size) * element


def kv_bytes_per_token(config, element):
    return 2 * config.kv_width * config.num_hidden_layers * element


def prefill_flops(config, lengths):
    """Flops of one step that runs whole prompts of these lengths (logits for the last token of each)."""
    c = config
    per_token = 2 * c.num_hidden_layers * ((c.q_width + 2 * c.kv_width) * c.hidden_size
                                            + c.hidden_size * c.q_width + 3 * c.intermediate_size * c.hidden_size)
    attention = sum(c.num_hidden_layers * 4 * c.q_width * t * (t + 1) // 2 for t in lengths)
    head = 2 * c.vocab_size * c.hidden_size * len(lengths)
    return per_token * sum(lengths) + attention + head


def sync():
    torch.cuda.synchronize()


def measured_ceilings(ops, device):
    """(GB/s of a kernel that only reads 2 GiB, TFLOP/s of bfloat16 matrix-core products on resident tiles of small
    whole numbers, the same on tiles of random numbers: the chip holds a lower clock on those)."""
    buffer = torch.ones(1 << 29, dtype=torch.int32, device=device)          # 2 GiB: beyond every cache
    best_read = 0.0
    for nontemporal in (False, True):
        ops.probe_read(buffer, nontemporal)
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record()
        count = sum(ops.probe_read(buffer, nontemporal) for _ in range(5))
        end.record()
        sync()
        best_read = max(best_read, count / (begin.elapsed_time(end) * 1e-3) / 1e9)
    del buffer
    rates = []
    for random_operands in (False, True):
        ops.probe_mfma(1000, device, random_operands)
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record()
        flops = ops.probe_mfma(200000, device, random_operands)
        end.record()
        sync()
        rates.append(flops / (begin.elapsed_time(end) * 1e-3) / 1e12)
    return best_read, rates[0], rates[1]


class Bench:
    def __init__(self, engine, seed):
        from xeno_rt_amd.sampling import Sampler, SamplerConfig
        from xeno_rt_amd.staging import staging_for
        self.staging = staging_for(engine.device)
        self.engine = engine
        self.sampler = Sampler(engine.ops, engine.device)
        self.greedy = SamplerConfig(temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0)
        self.generator = torch.Generator().manual_seed(seed)
        self.vocab = engine.config.vocab_size
        self.check = None

    def ids(self, count):
        return torch.randint(0, self.vocab, (count,), generator=self.generator).tolist()

    def fill(self, slots, length, chunk=2048):
        """Prefill every slot with `length` synthetic tokens, `chunk` tokens of one sequence per step."""
        for slot in slots:
            done = 0
            while done < length:
                count = min(chunk, length - done)
                self.engine.step([(slot, self.ids(count), [])])
                done += count
        sync()

    def decode(self, batch, steps, warmup, context, check=False):
        """Tokens per second, ms per step and the mean cache length of `steps` decode steps that end at `context` tokens."""
        engine = self.engine
        warmup = max(warmup, 1)            # the step that makes the first logits is not timed
        start_length = context - steps - warmup
        if start_length < 1:
            raise SystemExit(f"--steps {steps} + --warmup {warmup} do not fit a context of {context}")
        slots = [engine.alloc_slot() for _ in range(batch)]
        try:
            self.fill(slots, start_length)
            configs, histories, draws = [self.greedy] * batch, [[]] * batch, [0.0] * batch
            staging = self.staging
            entries = [(slot, row) for row, slot in enumerate(slots)]
            logits = engine.step([(slot, [token], [0]) for slot, token in zip(slots, self.ids(batch))])

            def one_step(logits):
                """As the generation loop does it: the next step starts from the sampled tokens on the
                device, and the host reads them while it runs."""
                drawn = self.sampler.launch(logits, configs, histories, draws)
                fetched = staging.fetch(drawn)
                logits = engine.step_from(drawn, entries)
                fetched.values()
                return logits

            for _ in range(warmup - 1):      # one warm-up step has been done above
                logits = one_step(logits)
            sync()
            begin = time.perf_counter()
            for _ in range(steps):
                logits = one_step(logits)
            sync()
            elapsed = time.perf_counter() - begin
            if check:
                self.check = self.compare_with_direct_step(slots)
            mean_length = start_length + warmup + (steps - 1) / 2.0 + 1     # keys each timed step reads, on average
            return batch * steps / elapsed, 1000.0 * elapsed / steps, mean_length
        finally:
            for slot in slots:
                engine.free_slot(slot)

    def compare_with_direct_step(self, slots):
        """The last token of every sequence once more (the cache rolled back by it), through the recorded graph
        and then, rolled back again, through kernels launched one by one on exactly the step's rows."""
        engine = self.engine
        tokens = self.ids(len(slots))
        step = [(slot, [token], [0]) for slot, token in zip(slots, tokens)]
        for slot in slots:
            engine.cache.truncate(slot, engine.length(slot) - 1)
        replayed = engine.step(step).clone()
        for slot in slots:
            engine.cache.truncate(slot, engine.length(slot) - 1)
        graphs, engine.graphs = engine.graphs, None
        try:
            direct = engine.step(step)
        finally:
            engine.graphs = graphs
        sync()
        scale = float(direct.abs().max())
        error = float((replayed - direct).abs().max()) / scale
        agree = float((replayed.argmax(dim=1) == direct.argmax(dim=1)).float().mean())
        limit = 2e-2 if engine.dtype == torch.bfloat16 else 2e-5
        return {"graph_vs_direct_max_err": round(error, 7), "limit": limit, "same_argmax": round(agree, 3),
                "finite": bool(torch.isfinite(replayed).all()), "ok": bool(error <= limit and torch.isfinite(replayed).all())}

    def prefill(self, lengths, repeats=3):
        """Best time of one step with whole prompts of these lengths into empty slots, logits of each last token."""
        best = None
        for _ in range(repeats + 1):
            slots = [self.engine.alloc_slot() for _ in lengths]
            step = [(slot, self.ids(n), [n - 1]) for slot, n in zip(slots, lengths)]
            sync()
            begin = time.perf_counter()
            self.engine.step(step)
            sync()
            elapsed = time.perf_counter() - begin
            for slot in slots:
                self.engine.free_slot(slot)
            best = elapsed if best is None else min(best, elapsed)     # the first run also warms up
        return best


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--shape", default="llama3-8b", choices=sorted(SHAPES))
    parser.add_argument("--batch", type=int, default=None, help="sequences of the headline decode step (8; 32 for qwen3-32b)")
    parser.add_argument("--layers", type=int, default=None,
                        help="run fewer layers of the same sizes (both numbers are reported)")
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    parser.add_argument("--context", type=int, default=CONTEXT,
                        help="tokens every sequence holds when the timed decode steps end (the headline: 4096)")
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--skip-points", action="store_true", help="only the headline batch")
    parser.add_argument("--phase", default="all", choices=["all", "decode", "prefill"],
                        help="for profiling: run only the decode steps, or only the prefill (prints a partial record)")
    parser.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS,
                        help="with --phase prefill: the prompt's length (the record's prefill is always of 2048 tokens)")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this library runs on a single MI355X)")
        return 2

    from xeno_rt_amd.config import parse_config
    from xeno_rt_amd.engine import Engine

    shape = SHAPES[args.shape]
    layers = args.layers if args.layers is not None else shape["num_hidden_layers"]
    batch = args.batch if args.batch is not None else HEADLINE_BATCH[args.shape]
    config = parse_config(dict(shape, num_hidden_layers=layers,
                               max_position_embeddings=max(shape["max_position_embeddings"], args.context, LONG_PREFILL)))
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    element = 2 if short == "bf16" else 4
    if args.phase != "all":
        args.skip_points = True
    others = () if args.skip_points else tuple(b for b in OTHER_BATCHES[args.shape] if b != batch)
    largest_batch = max((batch,) + others)
    context = args.context if args.phase != "prefill" else max(args.context, args.prefill_tokens)
    engine = Engine.random(config, seed=args.seed, dtype=args.dtype, max_tokens=largest_batch * context,
                           max_slots=largest_batch, max_context=context if args.skip_points else max(context, LONG_PREFILL))
    bench = Bench(engine, args.seed)

    def priced(ms, mean_length, sequences):
        step_bytes = weight_bytes(config, element) + sequences * mean_length * kv_bytes_per_token(config, element)
        return step_bytes / (ms * 1e-3) / 1e9

    if args.phase == "prefill":
        seconds = bench.prefill([args.prefill_tokens])
        print(json.dumps({"phase": "prefill", "tokens": args.prefill_tokens, "ms": round(seconds * 1e3, 3),
                          "frac": round(prefill_flops(config, [args.prefill_tokens]) / seconds / PEAK_FLOPS[short], 4)}), flush=True)
        return 0
    tokens_per_s, ms_per_step, mean_length = bench.decode(batch, args.steps, args.warmup, context, check=args.phase == "all")
    if args.phase == "decode":
        print(json.dumps({"phase": "decode", "batch": batch, "context": context, "ms_per_step": round(ms_per_step, 4),
                          "tokens_per_s": round(tokens_per_s, 1), "frac": round(priced(ms_per_step, mean_length, batch) / PEAK_HBM_GBS, 4)}), flush=True)
        return 0
    achieved = priced(ms_per_step, mean_length, batch)
    read_gbs, mfma_tflops, mfma_random_tflops = measured_ceilings(engine.ops, engine.device)

    seconds = bench.prefill([PREFILL_TOKENS])
    flops = prefill_flops(config, [PREFILL_TOKENS])
    prefill = {"value": round(PREFILL_TOKENS / seconds, 1), "tokens": PREFILL_TOKENS, "ms": round(seconds * 1e3, 3),
               "frac": round(flops / seconds / PEAK_FLOPS[short], 4)}
    if short == "bf16":
        prefill["measured_peak_tflops"] = round(mfma_tflops, 1)
        prefill["frac_of_measured"] = round(flops / seconds / (mfma_tflops * 1e12), 4)
        prefill["measured_peak_random_operands_tflops"] = round(mfma_random_tflops, 1)

    points = {}
    if not args.skip_points:
        for other in others:
            value, ms, length = bench.decode(other, args.steps, args.warmup, context)
            points[f"decode_b{other}"] = round(value, 1)
            points[f"decode_b{other}_ms"] = round(ms, 4)
            points[f"decode_b{other}_frac"] = round(priced(ms, length, other) / PEAK_HBM_GBS, 4)
        steps = min(args.steps, SHORT_CONTEXT - args.warmup - 2)
        value, ms, length = bench.decode(batch, steps, args.warmup, SHORT_CONTEXT)
        points[f"decode_b{batch}_ctx{SHORT_CONTEXT}"] = round(value, 1)
        points[f"decode_b{batch}_ctx{SHORT_CONTEXT}_ms"] = round(ms, 4)
        points[f"decode_b{batch}_ctx{SHORT_CONTEXT}_frac"] = round(priced(ms, length, batch) / PEAK_HBM_GBS, 4)
        if largest_batch * context >= LONG_PREFILL:
            seconds = bench.prefill([LONG_PREFILL], repeats=2)
            points[f"prefill_{LONG_PREFILL}"] = round(LONG_PREFILL / seconds, 1)
            points[f"prefill_{LONG_PREFILL}_ms"] = round(seconds * 1e3, 3)
            points[f"prefill_{LONG_PREFILL}_frac"] = round(prefill_flops(config, [LONG_PREFILL]) / seconds / PEAK_FLOPS[short], 4)
        if args.shape == "qwen3-8b":
            count, low, high = UNEQUAL_PROMPTS
            lengths = torch.randint(low, high + 1, (count,), generator=torch.Generator().manual_seed(args.seed)).tolist()
            seconds = bench.prefill(lengths)
            points["prefill_unequal_tokens"] = sum(lengths)
            points["prefill_unequal_ms"] = round(seconds * 1e3, 3)
            points["prefill_unequal"] = round(sum(lengths) / seconds, 1)
            points["prefill_unequal_frac"] = round(prefill_flops(config, lengths) / seconds / PEAK_FLOPS[short], 4)

    record = {
        "metric": "decode_tokens_per_s", "value": round(tokens_per_s, 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": short,
        "data": "synthetic token ids, random weights N(0, 0.02)",
        "config": {"model": MODEL_NAMES[args.shape], "layers_run": layers, "layers_of_shape": shape["num_hidden_layers"],
                   "hidden_size": config.hidden_size, "intermediate_size": config.intermediate_size,
                   "num_attention_heads": config.num_attention_heads, "num_key_value_heads": config.num_key_value_heads,
                   "head_dim": config.head_dim, "vocab_size": config.vocab_size, "rope_theta": config.rope_theta,
                   "rms_norm_eps": config.rms_norm_eps, "qk_norm": config.qk_norm, "global_batch": batch, "seq_len": context,
                   "prefill_tokens": PREFILL_TOKENS, "sampling": "greedy on device", "parallelism": "single GPU"},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4), "measured_peak": round(read_gbs, 1),
                     "frac_of_measured": round(achieved / read_gbs, 4)},
        "points": points,
        "check": bench.check,
    }
    print(json.dumps(record), flush=True)
    return 0 if bench.check is None or bench.check["ok"] else 1


if __name__ == "__main__":
    sys.exit(main())
