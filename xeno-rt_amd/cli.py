"""Command line, in the manner of the reference's `xrt generate`.

Options with the reference's names, defaults and meanings (crates/xrt-cli/src/main.rs:28-49):
--model, --max-tokens 128, --temperature 0.8, --top-k 40, --top-p 0.95,
--repetition-penalty 1.1, --seed. The reference takes --prompt as text and owns a
tokenizer; this library is driven by token ids: --prompt-ids "1,2,3" (repeat the option, or
separate prompts by ';', for a batch). Generated ids go to standard output, one line per
request; the reference's statistics line (main.rs:111-125) goes to standard error.
"""
from __future__ import annotations

import argparse
import sys
import time
from typing import List, Optional


def parse_prompts(values: List[str]) -> List[List[int]]:
    prompts = []
    for value in values:
        for part in value.split(";"):
            part = part.strip()
            prompts.append([int(t) for t in part.replace(",", " ").split()] if part else [])
    return prompts


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(prog="xrt", description="xeno-rt for MI355X: command line")
    commands = parser.add_subparsers(dest="command", required=True)
    gen = commands.add_parser("generate", help="generate token ids for one or more prompts")
    source = gen.add_mutually_exclusive_group(required=True)
    source.add_argument("--model", help="folder with config.json and model.safetensors")
    source.add_argument("--random", metavar="CONFIG_JSON", help="a config.json; weights are random, from --seed")
    gen.add_argument("--prompt-ids", action="append", required=True,
                     help="token ids of a prompt, e.g. 1,2,3; repeat or separate by ';' for a batch")
    gen.add_argument("--max-tokens", type=int, default=128)
    gen.add_argument("--temperature", type=float, default=0.8)
    gen.add_argument("--top-k", type=int, default=40)
    gen.add_argument("--top-p", type=float, default=0.95)
    gen.add_argument("--repetition-penalty", type=float, default=1.1)
    gen.add_argument("--seed", type=int, default=None)
    gen.add_argument("--stop-ids", default=None, help="stop token ids, e.g. 2,5 (default: eos_token_id of config.json)")
    gen.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32", "bf16", "fp32"])
    gen.add_argument("--batch-size", type=int, default=None, help="most requests that run together")
    gen.add_argument("--cache-tokens", type=int, default=None, help="tokens the cache holds (default: what the batch needs)")
    write = commands.add_parser("random-model", help="write a model folder with random weights")
    write.add_argument("--config", required=True, help="a config.json")
    write.add_argument("--out", required=True)
    write.add_argument("--seed", type=int, default=0)
    write.add_argument("--std", type=float, default=0.02)
    return parser


def run_generate(args) -> int:
    import json

    from .config import parse_config
    from .engine import GenerateRequest
    from .runtime import Runtime

    prompts = parse_prompts(args.prompt_ids)
    stops = None if args.stop_ids is None else [int(t) for t in args.stop_ids.replace(",", " ").split()]
    cache_tokens = args.cache_tokens
    if cache_tokens is None:
        from .cache import BLOCK_TOKENS          # requests hold the cache in whole blocks
        cache_tokens = sum(-(-(len(p) + max(1, args.max_tokens)) // BLOCK_TOKENS) * BLOCK_TOKENS for p in prompts) + BLOCK_TOKENS
    if args.model:
        runtime = Runtime.load(args.model, dtype=args.dtype, max_tokens=cache_tokens)
    else:
        with open(args.random) as handle:
            config = parse_config(json.load(handle))
        runtime = Runtime.random(config, seed=args.seed or 0, dtype=args.dtype, max_tokens=cache_tokens)
    requests = [GenerateRequest(p, max_tokens=args.max_tokens, temperature=args.temperature, top_k=args.top_k,
                                top_p=args.top_p, repetition_penalty=args.repetition_penalty, seed=args.seed,
                                stop_ids=stops) for p in prompts]
    first_token_at: Optional[float] = None
    count = 0
    start = time.perf_counter()

    def on_token(index: int, token: int) -> None:
        nonlocal first_token_at, count
        if first_token_at is None:
            first_token_at = time.perf_counter() - start
        count += 1

    results = runtime.new_session().generate_batch(requests, batch_size=args.batch_size, on_token=on_token)
    elapsed = time.perf_counter() - start
    for result in results:
        print(" ".join(str(t) for t in result.tokens), flush=True)
    prefill_ms = (first_token_at or 0.0) * 1000.0
    decode_time = elapsed - (first_token_at or 0.0)
    decode_rate = (count - 1) / decode_time if decode_time > 0 and count > 1 else 0.0
    total_rate = count / elapsed if elapsed > 0 else 0.0
    print(f"\n--- {count} tokens in {elapsed:.2f}s | prefill {prefill_ms:.0f}ms | decode {decode_rate:.2f} tok/s | "
          f"total {total_rate:.2f} tok/s ---", file=sys.stderr)
    return 0


def run_random_model(args) -> int:
    import json

    from .config import parse_config
    from .weights import write_random_model

    with open(args.config) as handle:
        config = parse_config(json.load(handle))
    print(write_random_model(config, args.out, seed=args.seed, std=args.std))
    return 0


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    if args.command == "generate":
        return run_generate(args)
    return run_random_model(args)


if __name__ == "__main__":
    sys.exit(main())
