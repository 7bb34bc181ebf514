"""The Python entry point, in the manner of the reference's runtime crate.

Reference: `Runtime::load` owns the model and hands out sessions
(crates/xrt-runtime/src/lib.rs:15-47); a `Session` generates for one request at a
time (`generate`, `generate_stream`, `reset`; crates/xrt-runtime/src/session.rs:45-69).
Here a runtime owns an engine (model, weights, cache, kernels); a session generates
for one request or for a batch of them, token ids in and token ids out (the
reference's tokenizer is not part of this library).
"""
from __future__ import annotations

from typing import Callable, List, Optional, Sequence

from .engine import Engine, GenerateRequest, GenerateResult, generate


class Runtime:
    def __init__(self, engine: Engine):
        self.engine = engine

    @classmethod
    def load(cls, model: str, dtype: str = "bfloat16", max_tokens: int = 8192, **options) -> "Runtime":
        """From a model folder (config.json + model.safetensors); lib.rs:21-30."""
        return cls(Engine.load(model, dtype=dtype, max_tokens=max_tokens, **options))

    @classmethod
    def random(cls, config, seed: int = 0, dtype: str = "bfloat16", max_tokens: int = 8192, **options) -> "Runtime":
        return cls(Engine.random(config, seed=seed, dtype=dtype, max_tokens=max_tokens, **options))

    @property
    def config(self):
        return self.engine.config

    def new_session(self) -> "Session":            # lib.rs:44-46
        return Session(self)


class Session:
    def __init__(self, runtime: Runtime):
        self.runtime = runtime

    def generate(self, request: GenerateRequest) -> List[int]:
        """The tokens generated for one request (session.rs:63-67)."""
        return self.generate_batch([request])[0].tokens

    def generate_stream(self, request: GenerateRequest, on_token: Callable[[int], None]) -> GenerateResult:
        """Like `generate`, calling on_token(token_id) as each token is produced (session.rs:69-72)."""
        return generate(self.runtime.engine, [request], on_token=lambda index, token: on_token(token))[0]

    def generate_batch(self, requests: Sequence[GenerateRequest], batch_size: Optional[int] = None,
                       on_token: Optional[Callable[[int, int], None]] = None) -> List[GenerateResult]:
        """All requests, in batches of at most batch_size that start together."""
        return generate(self.runtime.engine, requests, batch_size=batch_size, on_token=on_token)

    def reset(self) -> None:
        """Nothing is kept between calls: every request starts in an empty slot (session.rs:58-61)."""
        return None
