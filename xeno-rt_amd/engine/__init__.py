"""The engine: step function and generation loop."""
from .batch import StepBatch, build_batch
from .engine import Engine, StepError, compute_dtype
from .generate import GenerateRequest, GenerateResult, decide, generate, plan_batches, resolve_prompt

__all__ = ["StepBatch", "build_batch", "Engine", "StepError", "compute_dtype", "GenerateRequest",
           "GenerateResult", "decide", "generate", "plan_batches", "resolve_prompt"]
