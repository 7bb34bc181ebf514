"""Decode and prefill throughput of the Llama-3-8B-shaped model with random weights.

    python bench.py --gpus 1 --steps K --warmup W

A step is one decode step of the whole batch (8 sequences unless --batch says otherwise):
the engine's step function on one token per sequence, then greedy sampling on the device.
Every sequence's cache is first filled by real prefill steps so that the timed steps end at
the context length (4096). Beside the headline it measures one prefill of 2048 tokens and
decoding at batch 1 and 64, and prices the decode step against the HBM roofline (bytes it has
to read: every weight it uses once, plus the cache of the live sequences) and the prefill
against the dense bf16 MFMA peak. One JSON line goes to standard output.
"""
import argparse
import json
import sys
import time

import torch

PEAK_HBM_GBS = 8000.0           # MI355X HBM3E, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}   # dense MFMA, published

# BASELINE.json configs[2]: the Llama-3-8B shape
SHAPE = dict(architectures=["LlamaForCausalLM"], vocab_size=128256, hidden_size=4096, intermediate_size=14336,
             num_hidden_layers=32, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
             rms_norm_eps=1e-5, rope_theta=500000.0, max_position_embeddings=8192, tie_word_embeddings=False,
             hidden_act="silu", torch_dtype="bfloat16")
CONTEXT = 4096
PREFILL_TOKENS = 2048


def weight_bytes(config, element):
    """Bytes of every weight that one decode step reads once (embedding rows are negligible)."""
    c = config
    per_layer = (c.q_width + 2 * c.kv_width) * c.hidden_size + c.hidden_size * c.q_width \
        + 3 * c.intermediate_size * c.hidden_size + 2 * c.hidden_size
    return (c.num_hidden_layers * per_layer + c.hidden_size + c.vocab_size * c.hidden_size) * element


def kv_bytes_per_token(config, element):
    return 2 * config.kv_width * config.num_hidden_layers * element


def prefill_flops(config, tokens):
    c = config
    linear = 2 * tokens * c.num_hidden_layers * ((c.q_width + 2 * c.kv_width) * c.hidden_size
                                                  + c.hidden_size * c.q_width + 3 * c.intermediate_size * c.hidden_size)
    attention = c.num_hidden_layers * 4 * c.q_width * tokens * (tokens + 1) // 2
    head = 2 * c.vocab_size * c.hidden_size
    return linear + attention + head


def sync():
    torch.cuda.synchronize()


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

    def decode(self, batch, steps, warmup, context):
        """Tokens per second and ms per step of `steps` decode steps that end at `context` tokens."""
        engine = self.engine
        warmup = max(warmup, 1)            # the step that makes the first logits is not timed
        start_length = context - steps - warmup
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
            mean_length = start_length + warmup + (steps - 1) / 2.0 + 1     # keys each timed step reads, on average
            return batch * steps / elapsed, 1000.0 * elapsed / steps, mean_length
        finally:
            for slot in slots:
                engine.free_slot(slot)

    def prefill(self, tokens, repeats=3):
        """Best time of one whole prompt of `tokens` tokens into an empty slot, logits of the last token."""
        best = None
        for _ in range(repeats + 1):
            slot = self.engine.alloc_slot()
            ids = self.ids(tokens)
            sync()
            begin = time.perf_counter()
            self.engine.step([(slot, ids, [tokens - 1])])
            sync()
            elapsed = time.perf_counter() - begin
            self.engine.free_slot(slot)
            best = elapsed if best is None else min(best, elapsed)     # the first run also warms up
        return best


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--layers", type=int, default=SHAPE["num_hidden_layers"],
                        help="run fewer layers of the same sizes (both numbers are reported)")
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--skip-points", action="store_true", help="only the headline batch")
    parser.add_argument("--phase", default="all", choices=["all", "decode", "prefill"],
                        help="for profiling: run only the decode steps, or only the prefill (prints a partial record)")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this library runs on a single MI355X)")
        return 2

    from xeno_rt_amd.config import parse_config
    from xeno_rt_amd.engine import Engine

    raw = dict(SHAPE, num_hidden_layers=args.layers)
    config = parse_config(raw)
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    element = 2 if short == "bf16" else 4
    if args.phase != "all":
        args.skip_points = True
    largest_batch = args.batch if args.skip_points else max(args.batch, 64)
    engine = Engine.random(config, seed=args.seed, dtype=args.dtype, max_tokens=largest_batch * CONTEXT,
                           max_slots=largest_batch, max_context=CONTEXT)
    bench = Bench(engine, args.seed)

    if args.phase == "prefill":
        seconds = bench.prefill(PREFILL_TOKENS)
        print(json.dumps({"phase": "prefill", "tokens": PREFILL_TOKENS, "ms": round(seconds * 1e3, 3),
                          "frac": round(prefill_flops(config, PREFILL_TOKENS) / seconds / PEAK_FLOPS[short], 4)}), flush=True)
        return 0
    tokens_per_s, ms_per_step, mean_length = bench.decode(args.batch, args.steps, args.warmup, CONTEXT)
    if args.phase == "decode":
        print(json.dumps({"phase": "decode", "batch": args.batch, "ms_per_step": round(ms_per_step, 4),
                          "tokens_per_s": round(tokens_per_s, 1)}), flush=True)
        return 0
    step_bytes = weight_bytes(config, element) + args.batch * mean_length * kv_bytes_per_token(config, element)
    achieved = step_bytes / (ms_per_step * 1e-3) / 1e9

    seconds = bench.prefill(PREFILL_TOKENS)
    flops = prefill_flops(config, PREFILL_TOKENS)
    prefill = {"value": round(PREFILL_TOKENS / seconds, 1), "tokens": PREFILL_TOKENS, "ms": round(seconds * 1e3, 3),
               "frac": round(flops / seconds / PEAK_FLOPS[short], 4)}

    points = {}
    if not args.skip_points:
        for batch in (1, 64):
            value, _, _ = bench.decode(batch, args.steps, args.warmup, CONTEXT)
            points[f"decode_b{batch}"] = round(value, 1)

    record = {
        "metric": "decode_tokens_per_s", "value": round(tokens_per_s, 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": short,
        "data": "synthetic token ids, random weights N(0, 0.02)",
        "config": {"model": "Llama-3-8B shape", "layers_run": args.layers, "layers_of_shape": SHAPE["num_hidden_layers"],
                   "hidden_size": config.hidden_size, "intermediate_size": config.intermediate_size,
                   "num_attention_heads": config.num_attention_heads, "num_key_value_heads": config.num_key_value_heads,
                   "head_dim": config.head_dim, "vocab_size": config.vocab_size, "rope_theta": config.rope_theta,
                   "rms_norm_eps": config.rms_norm_eps, "global_batch": args.batch, "seq_len": CONTEXT,
                   "prefill_tokens": PREFILL_TOKENS, "sampling": "greedy on device", "parallelism": "single GPU"},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
        "points": points,
    }
    print(json.dumps(record), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
