"""MI355X-native model library for the Llama / Qwen3 dense decoder.

    from xeno_rt_amd import Runtime, GenerateRequest
    runtime = Runtime.load("model_folder", dtype="bfloat16")
    tokens = runtime.new_session().generate(GenerateRequest([1, 2, 3], max_tokens=16, temperature=0.0))
"""
from .engine import Engine, GenerateRequest, GenerateResult, StepError, generate
from .runtime import Runtime, Session
from .sampling import SamplerConfig

__all__ = ["Engine", "GenerateRequest", "GenerateResult", "StepError", "generate", "Runtime", "Session",
           "SamplerConfig"]
